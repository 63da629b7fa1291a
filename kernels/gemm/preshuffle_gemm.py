"""Same import path as the reference's kernels/gemm/preshuffle_gemm.py."""
from flydsl_amd.kernels.gemm.preshuffle_gemm import PreshuffleGemm, compile_preshuffle_gemm  # noqa: F401
