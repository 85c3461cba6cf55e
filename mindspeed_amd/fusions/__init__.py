"""Megatron-facing adapters (mirror of ``mindspeed.core.fusions`` for the expert path)."""
from .grouped_matmul import Ops, grouped_gemm_is_available, assert_grouped_gemm_is_available, get_device_capability  # noqa: F401
from .fused_moe_permute import permute, unpermute  # noqa: F401
