"""Expert dispatch either side of the routed-expert GEMMs: histogram, grouping by expert, gated combine."""

from kohakuwullm_amd.kernels.moe.moe_dispatch import combine_routed, expert_counts, expert_sort, expert_sort_into

__all__ = ["combine_routed", "expert_counts", "expert_sort", "expert_sort_into"]
