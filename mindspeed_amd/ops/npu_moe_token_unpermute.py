"""``npu_moe_token_unpermute`` on MI355X.

Mirrors mindspeed/ops/npu_moe_token_unpermute.py:13-22 and the autograd
Function of mindspeed/ops/csrc/cann/npu_moe_token_unpermute.cpp:95-148: same
signature, gradients to ``permuted_tokens`` and ``probs``.
"""
from __future__ import annotations

import torch

from .. import _lib, flop_counter

__all__ = ["npu_moe_token_unpermute"]


def _check_forward(permuted_tokens, sorted_indices, probs, padded_mode):
    # npu_moe_token_unpermute.cpp:31-62 (dtype widened from bf16-only).
    if padded_mode:
        raise RuntimeError("current version only support padded_mode is false")
    _lib.dtype_code(permuted_tokens.dtype, "Input tensor permuted_tokens")
    if sorted_indices.dtype != torch.int32:
        raise TypeError(f"Input tensor sorted_indices dtype [{sorted_indices.dtype}] is invalid, should be int32")
    if probs is not None:
        _lib.dtype_code(probs.dtype, "Input tensor probs")
    if permuted_tokens.dim() != 2:
        raise RuntimeError("The dims of input permuted_tokens should be 2 dimensional, "
                           f"but got {permuted_tokens.dim()}-dimensional.")
    if sorted_indices.dim() != 1:
        raise RuntimeError("The dims of input sorted_indices should be 1 dimensional, "
                           f"but got {sorted_indices.dim()}-dimensional.")
    if probs is not None and probs.dim() != 2:
        raise RuntimeError(f"The dims of input probs should be 2 dimensional, but got {probs.dim()}-dimensional.")
    _lib.require_device(permuted_tokens, "permuted_tokens")
    _lib.require_device(sorted_indices, "sorted_indices")
    if probs is not None:
        _lib.require_device(probs, "probs")


class _MoeTokenUnpermute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, permuted_tokens, sorted_indices, probs):
        lib = _lib.load()
        permuted_tokens = permuted_tokens.contiguous()
        sorted_indices = sorted_indices.contiguous()
        topk = 1 if probs is None else probs.size(1)
        if sorted_indices.size(0) % topk != 0:
            raise RuntimeError(f"sorted_indices has {sorted_indices.size(0)} entries, not a multiple of topk {topk}")
        num_tokens = sorted_indices.size(0) // topk  # npu_moe_token_unpermute.cpp:113
        if probs is not None:
            probs = probs.contiguous()
            if probs.size(0) != num_tokens:
                raise RuntimeError(f"probs has {probs.size(0)} rows, expected {num_tokens}")
        hidden = permuted_tokens.size(1)
        dev = permuted_tokens.device
        out = torch.empty((num_tokens, hidden), dtype=permuted_tokens.dtype, device=dev)
        work = flop_counter.unpermute_bytes(num_tokens, topk, hidden, permuted_tokens.element_size(),
                                            permuted_tokens.size(0))
        with torch.cuda.device(dev), flop_counter.op("unpermute", work, "byte", dev):
            _lib.check(lib.ms_moe_token_unpermute(
                _lib.stream_ptr(dev), _lib.ptr(permuted_tokens), _lib.ptr(sorted_indices), _lib.ptr(probs),
                num_tokens, topk, hidden, _lib.dtype_code(permuted_tokens.dtype, "permuted_tokens"),
                permuted_tokens.size(0), _lib.ptr(out)), "ms_moe_token_unpermute")
        ctx.save_for_backward(permuted_tokens, sorted_indices, probs)  # npu_moe_token_unpermute.cpp:117
        ctx.topk = topk
        ctx.num_tokens = num_tokens
        return out

    @staticmethod
    def backward(ctx, grad_out):
        permuted_tokens, sorted_indices, probs = ctx.saved_tensors
        lib = _lib.load()
        if grad_out.dim() != 2:
            raise RuntimeError("The dims of input unpermuted_tokens_grad should be 2 dimensional, "
                               f"but got {grad_out.dim()}-dimensional.")
        grad_out = grad_out.contiguous()
        dev = grad_out.device
        hidden = permuted_tokens.size(1)
        grad_permuted = torch.empty_like(permuted_tokens)  # npu_moe_token_unpermute.cpp:140
        grad_probs = torch.empty_like(probs) if probs is not None else None  # :141
        need_rows = ctx.num_tokens * ctx.topk
        if permuted_tokens.size(0) > need_rows:
            grad_permuted.zero_()
        work = flop_counter.unpermute_grad_bytes(ctx.num_tokens, ctx.topk, hidden, grad_out.element_size(),
                                                 permuted_tokens.size(0), probs is not None)
        with torch.cuda.device(dev), flop_counter.op("unpermute_grad", work, "byte", dev):
            _lib.check(lib.ms_moe_token_unpermute_grad(
                _lib.stream_ptr(dev), _lib.ptr(permuted_tokens), _lib.ptr(grad_out), _lib.ptr(sorted_indices),
                _lib.ptr(probs), ctx.num_tokens, ctx.topk, hidden,
                _lib.dtype_code(permuted_tokens.dtype, "permuted_tokens"), min(permuted_tokens.size(0), need_rows),
                _lib.ptr(grad_permuted), _lib.ptr(grad_probs)), "ms_moe_token_unpermute_grad")
        return grad_permuted, None, grad_probs


def npu_moe_token_unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor,
                            probs: torch.Tensor = None, padded_mode: bool = False,
                            restore_shape: torch.Size = None):
    """``out[t] = sum_j probs[t, j] * permuted_tokens[sorted_indices[t*topk+j]]``.

    ``sorted_indices`` is the int32 map returned by ``npu_moe_token_permute``;
    ``topk`` is ``probs.size(1)`` (1 without probs).  fp32 accumulation, one
    rounding.  ``restore_shape`` is accepted and ignored, as in the reference.
    """
    _check_forward(permuted_tokens, sorted_indices, probs, padded_mode)
    if probs is not None and probs.dtype != permuted_tokens.dtype:
        probs = probs.to(permuted_tokens.dtype)
    return _MoeTokenUnpermute.apply(permuted_tokens, sorted_indices, probs)
