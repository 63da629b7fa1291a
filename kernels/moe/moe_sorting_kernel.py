"""Same import path as the reference's kernels/moe/moe_sorting_kernel."""
from flydsl_amd.kernels.moe.moe_sorting import UNIT_SIZE, moe_sorting_flydsl, moe_sorting_get_workspace_size  # noqa: F401

__all__ = ["UNIT_SIZE", "moe_sorting_flydsl", "moe_sorting_get_workspace_size"]
