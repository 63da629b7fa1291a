"""Same import path as the reference's kernels/moe/moe_gemm_2stage."""
from flydsl_amd.kernels.moe.moe_gemm_2stage import compile_moe_gemm1, compile_moe_gemm2, compile_moe_reduction  # noqa: F401

__all__ = ["compile_moe_gemm1", "compile_moe_gemm2", "compile_moe_reduction"]
