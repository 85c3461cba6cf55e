"""``npu_moe_token_permute`` on MI355X.

Mirrors mindspeed/ops/npu_moe_token_permute.py:13-20 and the autograd
Function of mindspeed/ops/csrc/cann/npu_moe_token_permute.cpp:65-118: same
signature, same output shapes, gradient to ``tokens`` only.
"""
from __future__ import annotations

import torch

from .. import _lib
from ._kernels import K

__all__ = ["npu_moe_token_permute", "moe_token_permute_with_aux"]


def _check_forward(tokens, indices, padded_mode):
    # npu_moe_token_permute.cpp:31-51 (the dtype check is widened from bf16-only
    # to bf16/fp16/fp32: the torch path accepts any float dtype).
    if padded_mode:
        raise RuntimeError("current version only support padded_mode is false")
    _lib.dtype_code(tokens.dtype, "Input tensor tokens")
    _lib.index_code(indices.dtype, "Input tensor indices")
    if tokens.dim() != 2:
        raise RuntimeError(f"The dims of input tokens should be 2 dimensional, but got {tokens.dim()}-dimensional.")
    if indices.dim() not in (1, 2):
        raise RuntimeError(f"The dims of input indices should be 2 or 1 dimensional, but got {indices.dim()}-dimensional.")
    _lib.require_device(tokens, "tokens")
    _lib.require_device(indices, "indices")
    if indices.size(0) != tokens.size(0):
        raise RuntimeError(f"indices has {indices.size(0)} rows but tokens has {tokens.size(0)}")


def _actual_num_out(num_out_tokens, flatten_size):
    # npu_moe_token_permute.cpp:72,80
    n = 0 if num_out_tokens is None else int(num_out_tokens)
    return min(n, flatten_size) if n > 0 else n + flatten_size


def _permute_forward(tokens, indices, num_out, num_experts, want_sorted, want_counts):
    tokens = tokens.contiguous()
    indices = indices.contiguous()
    num_tokens, hidden = tokens.shape
    topk = 1 if indices.dim() == 1 else indices.size(1)
    flat = num_tokens * topk
    if not 0 <= num_out <= flat:
        raise RuntimeError(f"num_out_tokens resolves to {num_out}, outside [0, {flat}]")
    hint = 0 if num_experts is None else int(num_experts)
    if hint > _lib.MS_MAX_EXPERTS:
        raise RuntimeError(f"num_experts {hint} exceeds the sort's key range {_lib.MS_MAX_EXPERTS}")
    if hidden == 0:
        raise RuntimeError("tokens must have a non-empty hidden dimension")
    permuted, row_id_map, sorted_idx, counts = K.moe_token_permute(
        tokens, indices, num_out, hint, bool(want_sorted), bool(want_counts and hint > 0))
    return (permuted, row_id_map, sorted_idx if want_sorted else None,
            counts if (want_counts and hint > 0) else None, topk)


class _MoeTokenPermute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tokens, indices, num_out, num_experts, want_sorted, want_counts):
        permuted, row_id_map, sorted_idx, counts, topk = _permute_forward(
            tokens, indices, num_out, num_experts, want_sorted, want_counts)
        ctx.save_for_backward(row_id_map)
        ctx.set_materialize_grads(False)   # no zero-filled gradients for the integer outputs
        ctx.num_tokens = tokens.size(0)
        ctx.topk = topk
        outs = [permuted, row_id_map]
        ctx.mark_non_differentiable(row_id_map)
        if sorted_idx is not None:
            outs.append(sorted_idx)
            ctx.mark_non_differentiable(sorted_idx)
        if counts is not None:
            outs.append(counts)
            ctx.mark_non_differentiable(counts)
        return tuple(outs)

    @staticmethod
    def backward(ctx, grad_permuted, *_unused):
        (row_id_map,) = ctx.saved_tensors
        if grad_permuted is None:
            return None, None, None, None, None, None
        # npu_moe_token_permute.cpp:53-63,99-118
        if grad_permuted.dim() != 2:
            raise RuntimeError("The dims of input grad_permuted_tokens should be 2 dimensional, "
                               f"but got {grad_permuted.dim()}-dimensional.")
        grad_tokens = K.moe_token_permute_grad(grad_permuted.contiguous(), row_id_map, ctx.num_tokens, ctx.topk)
        return grad_tokens, None, None, None, None, None


def npu_moe_token_permute(tokens: torch.Tensor, indices: torch.Tensor, num_out_tokens: int = None,
                          padded_mode: bool = False):
    """Permute ``tokens`` so that rows of the same expert are contiguous.

    Returns ``(permuted_tokens, sorted_indices)``.  As in the reference's fused
    op, ``sorted_indices`` is the full-length int32 map that
    ``npu_moe_token_unpermute`` consumes: entry ``t*topk+j`` is the output row
    of that (token, slot) pair; entries ``>= permuted_tokens.size(0)`` are
    dropped rows.  Expert ids must lie in ``[0, 1024)``.
    """
    _check_forward(tokens, indices, padded_mode)
    num_out = _actual_num_out(num_out_tokens, indices.numel())
    permuted, row_id_map = _MoeTokenPermute.apply(tokens, indices, num_out, None, False, False)
    return permuted, row_id_map


def moe_token_permute_with_aux(tokens, indices, num_out_tokens=None, *, num_experts=None):
    """Same permute, plus the by-products the kernel has anyway.

    Returns ``(permuted_tokens, row_id_map, sorted_indices, tokens_per_expert)``
    where ``sorted_indices`` (int32, ``num_out`` long) is the order the torch
    path returns (mindspeed/core/transformer/moe/moe_utils.py:206-208) and
    ``tokens_per_expert`` (int64 ``[num_experts]``, or None without
    ``num_experts``) is ``bincount(indices)``.  ``num_experts`` also narrows
    the sort's key range.
    """
    _check_forward(tokens, indices, False)
    num_out = _actual_num_out(num_out_tokens, indices.numel())
    outs = _MoeTokenPermute.apply(tokens, indices, num_out, num_experts, True, num_experts is not None)
    permuted, row_id_map, sorted_idx = outs[0], outs[1], outs[2]
    counts = outs[3] if len(outs) > 3 else None
    return permuted, row_id_map, sorted_idx, counts
