"""``_GroupedMatmul`` / ``fused_grouped_matmul`` on MI355X.

Mirrors mindspeed/ops/grouped_matmul.py:10-82: the stacked-weight module API (``m_split`` per-group
counts, ``weights`` either ``[E, K, N]`` or ``[E, N, K]``) through which the lite / FSDP expert layers
reach the grouped matmul.  The reference slices the stack into E views and hands the list to
``torch_npu.npu_grouped_matmul``; here the stack is one strided operand of ``ms_gmm`` (transposed
weights are read in place), and the weight gradient is produced directly in the weights' own
orientation.
"""
from __future__ import annotations

import torch

from .gmm import _add_group_bias, gmm_raw

__all__ = ["_GroupedMatmul", "fused_grouped_matmul"]


class _GroupedMatmul(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input_tensor: torch.Tensor, weights, weights_bias, m_split, group_list_type) -> torch.Tensor:
        if not isinstance(m_split, torch.Tensor):   # grouped_matmul.py:13-17
            m_split = torch.tensor(list(m_split), device=input_tensor.device, dtype=torch.int64)
        ctx.group_list = m_split
        ctx.group_list_type = group_list_type
        if weights.dim() != 3:
            raise ValueError(f"weights must be [E, K, N] or [E, N, K], got {tuple(weights.shape)}")
        # grouped_matmul.py:26-36: [E, K, N] is used as it is, anything else is taken as [E, N, K]
        ctx.needs_transpose = weights.shape[1] != input_tensor.shape[-1]
        ctx.save_for_backward(input_tensor, weights)
        w = weights.transpose(1, 2) if ctx.needs_transpose else weights
        out = gmm_raw(input_tensor, w, ctx.group_list, 0, group_list_type)
        if weights_bias is not None:
            # grouped_matmul.py:40-42 hands `weights_bias` to the vendor op beside the list of weight slices: one [N]
            # vector per group (a stacked [E, N] tensor is taken too); no gradient flows to it (:80 returns None)
            bias = weights_bias if isinstance(weights_bias, torch.Tensor) else torch.stack(list(weights_bias))
            out = _add_group_bias(out, bias, ctx.group_list, group_list_type)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        inp, weights = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        # grouped_matmul.py:54-66: dX = dY @ W^T
        w_t = weights if ctx.needs_transpose else weights.transpose(1, 2)
        grad = gmm_raw(grad_output, w_t, ctx.group_list, 0, ctx.group_list_type)
        # grouped_matmul.py:68-78: dW[g] = x_g^T @ dY_g, returned in the orientation of `weights`
        if ctx.needs_transpose:
            grad_weight = gmm_raw(grad_output.t(), inp, ctx.group_list, 2, ctx.group_list_type)   # [E, N, K]
        else:
            grad_weight = gmm_raw(inp.t(), grad_output, ctx.group_list, 2, ctx.group_list_type)   # [E, K, N]
        return grad, grad_weight, None, None, None


def fused_grouped_matmul(inputs, m_split, weights):
    """grouped_matmul.py:81-82 (``group_list_type`` 1: ``m_split`` holds per-group counts)."""
    return _GroupedMatmul.apply(inputs, weights, None, m_split, 1)
