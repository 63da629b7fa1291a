"""Same import path as the reference's kernels/gemm/fp8_gemm_utils.py (the host helper only)."""
from flydsl_amd.layout import preshuffle_b  # noqa: F401
