"""Same import path as the reference's kernels/gemm/fp4_gemm_4wave.py."""
from flydsl_amd.kernels.gemm.fp4_gemm_4wave import compile_fp4_gemm_4w  # noqa: F401
