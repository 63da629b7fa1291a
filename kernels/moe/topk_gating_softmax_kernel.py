"""Same import path as the reference's kernels/moe/topk_gating_softmax_kernel."""
from flydsl_amd.kernels.moe.topk_gating_softmax import build_topk_gating_softmax_module  # noqa: F401

__all__ = ["build_topk_gating_softmax_module"]
