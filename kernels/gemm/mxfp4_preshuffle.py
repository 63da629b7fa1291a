"""Same import path as the reference's kernels/gemm/mxfp4_preshuffle.py."""
from flydsl_amd.kernels.gemm.mxfp4_preshuffle import launch_gemm  # noqa: F401
