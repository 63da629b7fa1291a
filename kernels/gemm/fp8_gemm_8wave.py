"""Same import path as the reference's kernels/gemm/fp8_gemm_8wave.py."""
from flydsl_amd.kernels.gemm.fp8_gemm_rowscale import compile_fp8_gemm_8w  # noqa: F401
