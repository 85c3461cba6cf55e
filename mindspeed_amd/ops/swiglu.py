"""Fused SwiGLU (+ per-row probability) on MI355X.

Mirrors ``fused_swiglu`` of mindspeed/core/fusions/fused_bias_swiglu.py:4-5
(``silu(x[..., :F]) * x[..., F:]``, autograd Function of
mindspeed/ops/csrc/atb/swiglu.cpp:64-126) and the probs product of
mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:41-44.
"""
from __future__ import annotations

import torch

from .. import _lib
from ._kernels import K

__all__ = ["fused_swiglu", "swiglu_with_probs"]


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, probs):
        _lib.require_device(x, "x")
        shape = x.shape
        if shape[-1] % 2 != 0:
            raise RuntimeError(f"the last dim of x must be even, got {shape[-1]}")
        ffn = shape[-1] // 2
        x2 = x.contiguous().view(-1, 2 * ffn)
        rows = x2.size(0)
        p = None
        if probs is not None:
            p = probs.contiguous().view(-1)
            if p.numel() != rows:
                raise RuntimeError(f"probs has {p.numel()} entries, expected {rows}")
            _lib.dtype_code(p.dtype, "probs")
        _lib.dtype_code(x.dtype, "x")
        y = K.swiglu(x2, p)
        ctx.save_for_backward(x2, p)
        ctx.x_shape = shape
        ctx.probs_shape = None if probs is None else probs.shape
        return y.view(*shape[:-1], ffn)

    @staticmethod
    def backward(ctx, grad_y):
        x2, p = ctx.saved_tensors
        rows, two_ffn = x2.shape
        gx, gp = K.swiglu_grad(grad_y.contiguous().view(rows, two_ffn // 2), x2, p)
        return gx.view(ctx.x_shape), (gp.view(ctx.probs_shape) if p is not None else None)


def fused_swiglu(x):
    return _SwiGLU.apply(x, None)


def swiglu_with_probs(x, probs):
    """``silu(gate) * up * probs[:, None]`` cast to ``x.dtype`` (experts.py:41-44)."""
    return _SwiGLU.apply(x, probs)
