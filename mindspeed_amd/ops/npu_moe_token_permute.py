"""``npu_moe_token_permute`` on MI355X.

Mirrors mindspeed/ops/npu_moe_token_permute.py:13-20 and the autograd
Function of mindspeed/ops/csrc/cann/npu_moe_token_permute.cpp:65-118: same
signature, same output shapes, gradient to ``tokens`` only.
"""
from __future__ import annotations

import torch

from .. import _lib, flop_counter

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
    lib = _lib.load()
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
    dev = tokens.device
    row_id_map = torch.empty(flat, dtype=torch.int32, device=dev)
    permuted = torch.empty((num_out, hidden), dtype=tokens.dtype, device=dev)
    sorted_idx = torch.empty(num_out, dtype=torch.int32, device=dev) if want_sorted else None
    counts = torch.empty(hint, dtype=torch.int64, device=dev) if (want_counts and hint > 0) else None
    if hidden == 0:
        raise RuntimeError("tokens must have a non-empty hidden dimension")
    import ctypes
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_moe_token_permute_workspace_size(num_tokens, topk, hint, ctypes.byref(nbytes)),
               "ms_moe_token_permute_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    work = flop_counter.permute_bytes(num_tokens, topk, hidden, tokens.element_size(), indices.element_size(), num_out)
    with torch.cuda.device(dev), flop_counter.op("permute", work, "byte", dev):
        _lib.check(lib.ms_moe_token_permute(
            _lib.stream_ptr(dev), _lib.ptr(tokens), _lib.ptr(indices), _lib.index_code(indices.dtype, "indices"),
            num_tokens, topk, hidden, _lib.dtype_code(tokens.dtype, "tokens"), num_out, hint,
            _lib.ptr(permuted), _lib.ptr(row_id_map), _lib.ptr(sorted_idx), _lib.ptr(counts),
            _lib.ptr(ws), ws.numel()), "ms_moe_token_permute")
    return permuted, row_id_map, sorted_idx, counts, topk


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
        grad_permuted = grad_permuted.contiguous()
        lib = _lib.load()
        dev = grad_permuted.device
        hidden = grad_permuted.size(1)
        grad_tokens = torch.empty((ctx.num_tokens, hidden), dtype=grad_permuted.dtype, device=dev)
        work = flop_counter.permute_grad_bytes(ctx.num_tokens, ctx.topk, hidden, grad_permuted.element_size(),
                                               grad_permuted.size(0))
        with torch.cuda.device(dev), flop_counter.op("permute_grad", work, "byte", dev):
            _lib.check(lib.ms_moe_token_permute_grad(
                _lib.stream_ptr(dev), _lib.ptr(grad_permuted), _lib.ptr(row_id_map), ctx.num_tokens, ctx.topk,
                hidden, _lib.dtype_code(grad_permuted.dtype, "grad_permuted_tokens"), grad_permuted.size(0),
                _lib.ptr(grad_tokens)), "ms_moe_token_permute_grad")
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
