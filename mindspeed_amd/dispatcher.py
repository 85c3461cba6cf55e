"""Single-rank ``dispatch_mlp_combine``: permute -> grouped MLP -> weighted unpermute.

Mirrors mindspeed/fsdp/distributed/expert_parallel/dispatcher.py:37-52,81-113 for
one rank (``ep_size == 1``: no all-to-all, and the second permute / unpermute
pair of the reference is the identity because rows are already expert-major).
``tokens_per_expert`` comes out of the permute kernel's histogram instead of a
separate ``torch.bincount`` (dispatcher.py:64), and stays on the device.
"""
from __future__ import annotations

import torch

from .ops import (fused_swiglu, grouped_mlp, moe_token_permute_with_aux, npu_gmm_v2, npu_moe_token_unpermute)

__all__ = ["experts_computation", "dispatch_mlp_combine"]


def _fusable(hidden_states, gate_up_weights, down_weights):
    """Whether the fused matmul + SwiGLU kernels take these operands (16-bit, vector-access layout)."""
    ffn = gate_up_weights.size(-1) // 2
    return (hidden_states.dtype in (torch.bfloat16, torch.float16) and gate_up_weights.dim() == 3
            and down_weights.dim() == 3 and down_weights.dtype == hidden_states.dtype
            and hidden_states.size(-1) % 8 == 0 and ffn % 8 == 0 and gate_up_weights.size(-1) % 2 == 0
            and down_weights.size(-1) % 8 == 0 and down_weights.size(1) == ffn
            and hidden_states.data_ptr() % 16 == 0 and gate_up_weights.data_ptr() % 16 == 0
            and down_weights.data_ptr() % 16 == 0)


def experts_computation(hidden_states, split_list, gate_up_weights, down_weights, fuse_activation=None,
                        gemm_fusion=False):
    """``gmm -> silu(gate) * up -> gmm`` (dispatcher.py:93-104); ``split_list`` = rows per expert.

    The default (``fuse_activation=None``) is the reference's op sequence, one kernel per op, wherever a backward pass
    may follow; under ``torch.no_grad()`` it is the fused form, whose values are the same bit for bit and which then
    skips the fc1 output (2 % faster per forward pass on the Mixtral shape).  With ``fuse_activation`` the activation
    comes out of the first grouped matmul's epilogue and its backward rides on the epilogue of the second
    matmul's dX product (same values as the separate kernels', same step time, one buffer and two launches
    fewer) whenever the operands allow it.  ``gemm_fusion``: the weight gradients are added into the weights' fp32
    ``main_grad`` by the weight-gradient product itself (mindspeed/ops/gmm.py:56-89; one kernel per op then)."""
    if gemm_fusion:
        fc1 = npu_gmm_v2(hidden_states, gate_up_weights, group_list=split_list, group_type=0, gemm_fusion=True,
                         original_weight=gate_up_weights)
        return npu_gmm_v2(fused_swiglu(fc1), down_weights, group_list=split_list, group_type=0, gemm_fusion=True,
                          original_weight=down_weights)
    if fuse_activation is None:
        fuse_activation = not torch.is_grad_enabled()
    if fuse_activation and _fusable(hidden_states, gate_up_weights, down_weights):
        return grouped_mlp(hidden_states, gate_up_weights, down_weights, split_list)
    fc1 = npu_gmm_v2(hidden_states, gate_up_weights, group_list=split_list, group_type=0)
    act = fused_swiglu(fc1)
    return npu_gmm_v2(act, down_weights, group_list=split_list, group_type=0)


def dispatch_mlp_combine(hidden_states, top_k_index, top_k_weights, weights, num_global_experts=None,
                         fuse_activation=None, gemm_fusion=False):
    gate_up_weights, down_weights = weights
    num_experts = gate_up_weights.size(0) if num_global_experts is None else num_global_experts
    permuted, row_id_map, _, tokens_per_expert = moe_token_permute_with_aux(
        hidden_states, top_k_index, num_experts=num_experts)
    out = experts_computation(permuted, tokens_per_expert, gate_up_weights, down_weights, fuse_activation, gemm_fusion)
    return npu_moe_token_unpermute(out, row_id_map, top_k_weights)
