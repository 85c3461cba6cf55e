"""Routing-map ``permute`` / ``unpermute`` hooks under the reference's module name
(mindspeed/core/fusions/fused_moe_permute.py:50-85, substituted for Megatron's ``moe_utils.permute`` /
``unpermute`` by mindspeed/features_manager/fusions/fused_moe_permute.py:77-90)."""
from ..ops.moe_permute_mask_map import permute, unpermute  # noqa: F401
from ..ops.sort_chunks import sort_chunks_by_idxs  # noqa: F401
