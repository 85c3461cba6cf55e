"""Fused SwiGLU (+ per-row probability) on MI355X.

Mirrors ``fused_swiglu`` of mindspeed/core/fusions/fused_bias_swiglu.py:4-5
(``silu(x[..., :F]) * x[..., F:]``, autograd Function of
mindspeed/ops/csrc/atb/swiglu.cpp:64-126) and the probs product of
mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:41-44.
"""
from __future__ import annotations

import torch

from .. import _lib, flop_counter

__all__ = ["fused_swiglu", "swiglu_with_probs"]


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, probs):
        lib = _lib.load()
        _lib.require_device(x, "x")
        shape = x.shape
        if shape[-1] % 2 != 0:
            raise RuntimeError(f"the last dim of x must be even, got {shape[-1]}")
        ffn = shape[-1] // 2
        x2 = x.contiguous().view(-1, 2 * ffn)
        rows = x2.size(0)
        p = None
        p_code = 0
        if probs is not None:
            p = probs.contiguous().view(-1)
            if p.numel() != rows:
                raise RuntimeError(f"probs has {p.numel()} entries, expected {rows}")
            p_code = _lib.dtype_code(p.dtype, "probs")
        y = torch.empty((rows, ffn), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device), flop_counter.op(
                "swiglu", flop_counter.swiglu_bytes(rows, ffn, x.element_size()), "byte", x.device):
            _lib.check(lib.ms_swiglu(_lib.stream_ptr(x.device), _lib.ptr(x2), _lib.ptr(p), p_code, rows, ffn,
                                     _lib.dtype_code(x.dtype, "x"), _lib.ptr(y)), "ms_swiglu")
        ctx.save_for_backward(x2, p)
        ctx.x_shape = shape
        ctx.probs_shape = None if probs is None else probs.shape
        return y.view(*shape[:-1], ffn)

    @staticmethod
    def backward(ctx, grad_y):
        x2, p = ctx.saved_tensors
        lib = _lib.load()
        rows, two_ffn = x2.shape
        ffn = two_ffn // 2
        g = grad_y.contiguous().view(rows, ffn)
        gx = torch.empty_like(x2)
        gp = torch.empty_like(p) if p is not None else None
        p_code = _lib.dtype_code(p.dtype, "probs") if p is not None else 0
        with torch.cuda.device(x2.device), flop_counter.op(
                "swiglu_grad", flop_counter.swiglu_bytes(rows, ffn, x2.element_size(), True), "byte", x2.device):
            _lib.check(lib.ms_swiglu_grad(_lib.stream_ptr(x2.device), _lib.ptr(g), _lib.ptr(x2), _lib.ptr(p), p_code,
                                          rows, ffn, _lib.dtype_code(x2.dtype, "x"), _lib.ptr(gx), _lib.ptr(gp)),
                       "ms_swiglu_grad")
        return gx.view(ctx.x_shape), (gp.view(ctx.probs_shape) if gp is not None else None)


def fused_swiglu(x):
    return _SwiGLU.apply(x, None)


def swiglu_with_probs(x, probs):
    """``silu(gate) * up * probs[:, None]`` cast to ``x.dtype`` (experts.py:41-44)."""
    return _SwiGLU.apply(x, probs)
