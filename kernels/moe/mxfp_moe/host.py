"""Same import path as the reference's kernels/moe/mxfp_moe/host."""
from flydsl_amd.kernels.moe.mxfp_moe import flydsl_mxfp4_gemm1, flydsl_mxfp4_gemm2  # noqa: F401

__all__ = ["flydsl_mxfp4_gemm1", "flydsl_mxfp4_gemm2"]
