"""Same import path as the reference's kernels/moe/moe_sorting_kernel."""
from flydsl_amd.kernels.moe.moe_sorting import (  # noqa: F401
    UNIT_SIZE,
    moe_softmax_sort_flydsl,
    moe_sorting_flydsl,
    moe_sorting_get_workspace_size,
)

__all__ = ["UNIT_SIZE", "moe_softmax_sort_flydsl", "moe_sorting_flydsl", "moe_sorting_get_workspace_size"]
