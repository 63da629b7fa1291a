"""Same import path as the reference's kernels/moe/mxfp_moe."""
from flydsl_amd.kernels.moe.mxfp_moe import flydsl_mxfp4_gemm1, flydsl_mxfp4_gemm2, gemm1_grid, moe_mxfp4_sort  # noqa: F401

__all__ = ["flydsl_mxfp4_gemm1", "flydsl_mxfp4_gemm2", "gemm1_grid", "moe_mxfp4_sort"]
