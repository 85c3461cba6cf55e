"""Grouped matmul with the SwiGLU (x probability) activation fused into its epilogue.

The reference runs three ops in a row in ``GmmExpertsImpl.forward``
(mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:113-127): ``fc1 = gmm(x, w1)``,
``act = (fused_swiglu(fc1) * probs).to(dtype)`` (:41-44), then ``gmm(act, w2)``; with activation
recomputation the activation is dropped after the second matmul and rebuilt from ``fc1`` in backward
(:121-127,183-191).  Here the first two are one kernel launch: every tile of the first grouped matmul
holds 128 gate columns and the matching 128 up columns, and its epilogue writes both the fc1 output (kept
for backward, exactly as the reference keeps it) and the activation, computed from the already rounded
fc1 values — bit for bit what the stand-alone SwiGLU kernel produces from the stored fc1 output.

Backward is the reference's: SwiGLU backward on the saved fc1 output (which also yields the gradient of
the probabilities), then dX and dW of the grouped matmul.  ``recompute_activation=True`` keeps only the
fc1 output alive, as ``CheckpointWithoutOutput`` does; the activation handed to the caller is then simply
not saved for backward (nothing in this function's backward needs it).
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib, flop_counter
from .gmm import _beside, _group_list_tensor, gmm_raw

__all__ = ["gmm_swiglu", "GmmSwigluFunction"]


def _gmm_swiglu_forward(x, weight, group_list, group_list_type, probs):
    lib = _lib.load()
    _lib.require_device(x, "x")
    _lib.require_device(weight, "weight")
    if x.dim() != 2 or weight.dim() != 3 or weight.size(1) != x.size(1) or weight.size(2) % 2 != 0:
        raise ValueError(f"need x [M, K] and weight [E, K, 2*ffn], got {tuple(x.shape)}, {tuple(weight.shape)}")
    if weight.dtype != x.dtype:
        raise TypeError(f"x and weight must have the same dtype, got {x.dtype} and {weight.dtype}")
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"gmm_swiglu computes in bf16 or fp16, got {x.dtype}")
    dev = x.device
    x = x.contiguous()
    weight = weight.contiguous()
    gl = _group_list_tensor(group_list, dev)
    if gl.dtype != torch.int64 or gl.dim() != 1 or gl.numel() != weight.size(0):
        raise TypeError("group_list must be a one-dimensional int64 tensor with one entry per expert")
    m, k = x.shape
    ffn = weight.size(2) // 2
    p = None
    p_code = 0
    if probs is not None:
        _lib.require_device(probs, "probs")
        p = probs.contiguous().view(-1)
        if p.numel() != m:
            raise RuntimeError(f"probs has {p.numel()} entries, expected {m}")
        p_code = _lib.dtype_code(p.dtype, "probs")
    fc1 = torch.empty((m, 2 * ffn), dtype=x.dtype, device=dev)
    act = torch.empty((m, ffn), dtype=x.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_gmm_workspace_size(gl.numel(), m, 0, ctypes.byref(nbytes)), "ms_gmm_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    with torch.cuda.device(dev), flop_counter.op("gmm_fwd", flop_counter.gmm_flops(m, k, 2 * ffn), "flop", dev):
        _lib.check(lib.ms_gmm_swiglu(
            _lib.stream_ptr(dev), _lib.ptr(x), x.stride(0), x.stride(1), _lib.ptr(weight), weight.stride(0),
            weight.stride(1), weight.stride(2), _lib.ptr(fc1), 2 * ffn, _lib.ptr(act), ffn, _lib.ptr(p), p_code,
            _lib.ptr(gl), group_list_type, gl.numel(), m, k, ffn, _lib.dtype_code(x.dtype, "x"), _lib.ptr(ws),
            ws.numel()), "ms_gmm_swiglu")
    return fc1, act, gl, p


class GmmSwigluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, group_list, group_list_type, probs):
        fc1, act, gl, p = _gmm_swiglu_forward(x, weight, group_list, group_list_type, probs)
        ctx.save_for_backward(x, weight, gl, fc1, p)
        ctx.group_list_type = group_list_type
        ctx.probs_shape = None if probs is None else probs.shape
        return act

    @staticmethod
    def backward(ctx, grad_act):
        x, weight, gl, fc1, p = ctx.saved_tensors
        lib = _lib.load()
        dev = grad_act.device
        rows, two_ffn = fc1.shape
        ffn = two_ffn // 2
        g = grad_act.contiguous()
        d_fc1 = torch.empty_like(fc1)
        gp = torch.empty_like(p) if p is not None else None
        p_code = _lib.dtype_code(p.dtype, "probs") if p is not None else 0
        with torch.cuda.device(dev), flop_counter.op(
                "swiglu_grad", flop_counter.swiglu_bytes(rows, ffn, fc1.element_size(), True), "byte", dev):
            _lib.check(lib.ms_swiglu_grad(_lib.stream_ptr(dev), _lib.ptr(g), _lib.ptr(fc1), _lib.ptr(p), p_code, rows,
                                          ffn, _lib.dtype_code(fc1.dtype, "x"), _lib.ptr(d_fc1), _lib.ptr(gp)),
                       "ms_swiglu_grad")
        glt = ctx.group_list_type
        dx = dw = None
        if ctx.needs_input_grad[1]:
            dw = torch.empty(weight.shape, dtype=weight.dtype, device=dev)
            with _beside(dev) as side:
                gmm_raw(x.t(), d_fc1, gl, 2, glt, out=dw)
            if ctx.needs_input_grad[0]:
                dx = gmm_raw(d_fc1, weight.transpose(1, 2), gl, 0, glt)
            side.join()
        elif ctx.needs_input_grad[0]:
            dx = gmm_raw(d_fc1, weight.transpose(1, 2), gl, 0, glt)
        gp_out = gp.view(ctx.probs_shape) if (gp is not None and ctx.needs_input_grad[4]) else None
        return dx, dw, None, None, gp_out


def gmm_swiglu(x, weight, group_list, probs=None, *, group_list_type: int = 1):
    """``silu(fc1[:, :ffn]) * fc1[:, ffn:] * probs[:, None]`` with ``fc1 = grouped_matmul(x, weight)``.

    ``x [M, K]``, ``weight [E, K, 2*ffn]`` (gate columns first), ``group_list`` int64 ``[E]`` (per-expert row
    counts with ``group_list_type`` 1, cumulative offsets with 0), ``probs`` optional ``[M]`` / ``[M, 1]``.
    Needs the vector-access layout (16-byte aligned tensors, ``K`` and ``ffn`` multiples of 8); otherwise the
    library reports it and the caller can run ``npu_gmm`` and ``swiglu_with_probs`` one after the other.
    """
    return GmmSwigluFunction.apply(x, weight, group_list, group_list_type, probs)
