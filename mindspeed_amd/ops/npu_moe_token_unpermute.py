"""``npu_moe_token_unpermute`` on MI355X.

Mirrors mindspeed/ops/npu_moe_token_unpermute.py:13-22 and the autograd
Function of mindspeed/ops/csrc/cann/npu_moe_token_unpermute.cpp:95-148: same
signature, gradients to ``permuted_tokens`` and ``probs``.
"""
from __future__ import annotations

import torch

from .. import _lib
from ._kernels import K

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
        out = K.moe_token_unpermute(permuted_tokens, sorted_indices, probs, num_tokens, topk)
        ctx.save_for_backward(permuted_tokens, sorted_indices, probs)  # npu_moe_token_unpermute.cpp:117
        ctx.topk = topk
        ctx.num_tokens = num_tokens
        return out

    @staticmethod
    def backward(ctx, grad_out):
        permuted_tokens, sorted_indices, probs = ctx.saved_tensors
        if grad_out.dim() != 2:
            raise RuntimeError("The dims of input unpermuted_tokens_grad should be 2 dimensional, "
                               f"but got {grad_out.dim()}-dimensional.")
        # grad_permuted has the shape of permuted_tokens, grad_probs that of probs (npu_moe_token_unpermute.cpp:140-141);
        # rows of permuted_tokens that no (token, slot) pair maps to get zeros
        grad_permuted, grad_probs = K.moe_token_unpermute_grad(
            permuted_tokens, grad_out.contiguous(), sorted_indices, probs, ctx.num_tokens, ctx.topk,
            permuted_tokens.size(0))
        return grad_permuted, None, (grad_probs if probs is not None else None)


def npu_moe_token_unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor,
                            probs: torch.Tensor = None, padded_mode: bool = False,
                            restore_shape: torch.Size = None):
    """``out[t] = sum_j probs[t, j] * permuted_tokens[sorted_indices[t*topk+j]]``.

    ``sorted_indices`` is the int32 map returned by ``npu_moe_token_permute``;
    ``topk`` is ``probs.size(1)`` (1 without probs).  ``probs`` may have a dtype of
    their own (fp32 router probabilities beside bf16 tokens): they are used
    unrounded, and their gradient comes back in that dtype.  fp32 accumulation, one
    rounding to the tokens' dtype.  ``restore_shape`` is accepted and ignored, as
    in the reference.
    """
    _check_forward(permuted_tokens, sorted_indices, probs, padded_mode)
    return _MoeTokenUnpermute.apply(permuted_tokens, sorted_indices, probs)
