"""Grouped matmul with the SwiGLU (x probability) activation fused into its epilogue.

The reference runs three ops in a row in ``GmmExpertsImpl.forward``
(mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:113-127): ``fc1 = gmm(x, w1)``,
``act = (fused_swiglu(fc1) * probs).to(dtype)`` (:41-44), then ``gmm(act, w2)``; with activation
recomputation the activation is dropped after the second matmul and rebuilt from ``fc1`` in backward
(:121-127,183-191).  Here the first two are one kernel launch: every tile of the first grouped matmul
holds 128 gate columns and the matching 128 up columns, and its epilogue writes both the fc1 output (kept
for backward, exactly as the reference keeps it) and the activation, computed from the already rounded
fc1 values — bit for bit what the stand-alone SwiGLU kernel produces from the stored fc1 output.  Where
nothing is differentiated (inference, ``torch.no_grad()``) the fc1 output is not written at all.

Backward is the reference's: SwiGLU backward on the saved fc1 output (which also yields the gradient of
the probabilities), then dX and dW of the grouped matmul.  ``recompute_activation=True`` keeps only the
fc1 output alive, as ``CheckpointWithoutOutput`` does; the activation handed to the caller is then simply
not saved for backward (nothing in this function's backward needs it).
"""
from __future__ import annotations

import torch

from .. import _lib
from ._kernels import K
from .gmm import _beside, _group_list_tensor, gmm_raw

__all__ = ["gmm_swiglu", "GmmSwigluFunction", "grouped_mlp", "GroupedMLPFunction"]


def _gmm_swiglu_forward(x, weight, group_list, group_list_type, probs, want_fc1=True):
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
    m = x.size(0)
    p = None
    if probs is not None:
        _lib.require_device(probs, "probs")
        p = probs.contiguous().view(-1)
        if p.numel() != m:
            raise RuntimeError(f"probs has {p.numel()} entries, expected {m}")
        _lib.dtype_code(p.dtype, "probs")
    fc1, act = K.gmm_swiglu(x, weight, gl, group_list_type, p, want_fc1)
    return (fc1 if want_fc1 else None), act, gl, p


class GmmSwigluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, group_list, group_list_type, probs, differentiated=True):
        # the fc1 output exists for the backward pass only: where nothing is differentiated (inference) it is not
        # stored.  The caller decides (see _differentiated): ctx.needs_input_grad mirrors the inputs' requires_grad
        # whatever the grad mode, so it cannot tell torch.no_grad() from training.
        fc1, act, gl, p = _gmm_swiglu_forward(x, weight, group_list, group_list_type, probs, want_fc1=differentiated)
        if differentiated:
            ctx.save_for_backward(x, weight, gl, fc1, p)
        ctx.group_list_type = group_list_type
        ctx.probs_shape = None if probs is None else probs.shape
        return act

    @staticmethod
    def backward(ctx, grad_act):
        x, weight, gl, fc1, p = ctx.saved_tensors
        dev = grad_act.device
        d_fc1, gp = _swiglu_grad_from_fc1(grad_act.contiguous(), fc1, p)
        glt = ctx.group_list_type
        dx = dw = None
        if ctx.needs_input_grad[1]:
            dw = torch.empty(weight.shape, dtype=weight.dtype, device=dev)
            with _beside(d_fc1) as side:
                gmm_raw(x.t(), d_fc1, gl, 2, glt, out=dw)
            if ctx.needs_input_grad[0]:
                dx = gmm_raw(d_fc1, weight.transpose(1, 2), gl, 0, glt)
            side.join()
        elif ctx.needs_input_grad[0]:
            dx = gmm_raw(d_fc1, weight.transpose(1, 2), gl, 0, glt)
        gp_out = gp.view(ctx.probs_shape) if (gp is not None and ctx.needs_input_grad[4]) else None
        return dx, dw, None, None, gp_out, None


def _differentiated(*tensors) -> bool:
    """Whether autograd will record the call: grad mode on and some input asks for a gradient."""
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def gmm_swiglu(x, weight, group_list, probs=None, *, group_list_type: int = 1):
    """``silu(fc1[:, :ffn]) * fc1[:, ffn:] * probs[:, None]`` with ``fc1 = grouped_matmul(x, weight)``.

    ``x [M, K]``, ``weight [E, K, 2*ffn]`` (gate columns first), ``group_list`` int64 ``[E]`` (per-expert row
    counts with ``group_list_type`` 1, cumulative offsets with 0), ``probs`` optional ``[M]`` / ``[M, 1]``.
    Needs the vector-access layout (16-byte aligned tensors, ``K`` and ``ffn`` multiples of 8); otherwise the
    library reports it and the caller can run ``npu_gmm`` and ``swiglu_with_probs`` one after the other.
    """
    return GmmSwigluFunction.apply(x, weight, group_list, group_list_type, probs, _differentiated(x, weight, probs))


def _swiglu_from_fc1(fc1, p):
    """The activation again from the saved fc1 output (the recomputation of experts.py:183-191)."""
    return K.swiglu(fc1, p)


def _swiglu_grad_from_fc1(dact, fc1, p):
    d_fc1, gp = K.swiglu_grad(dact, fc1, p)
    return d_fc1, (gp if p is not None else None)


class GroupedMLPFunction(torch.autograd.Function):
    """The whole expert MLP of ``GmmExpertsImpl.forward`` (experts.py:113-160) as one autograd node:

    forward   ``fc1 = gmm(x, w1)``; ``act = silu(gate) * up * probs``; ``out = gmm(act, w2)``
    backward  ``dact = dy @ w2^T``; ``d_fc1, d_probs = SwiGLU backward on the saved fc1``;
              ``dW2 = act^T dy``; ``dx = d_fc1 @ w1^T``; ``dW1 = x^T d_fc1``

    With ``MINDSPEED_AMD_OVERLAP_WGRAD=1`` one node instead of three keeps a second stream busy from start to end
    of the backward pass: dW2 runs beside dX2 and the SwiGLU backward, dW1 beside dX1, with one join at the very
    end (measured on the Mixtral shape this is no faster than three nodes that each overlap their own dW, nor than
    no overlap at all: the step is limited by board power, not by idle units).
    ``fused_kernels``: the activation comes out of the first matmul's epilogue and its backward rides on the
    epilogue of the dX2 product (16-bit, vector-access layout only); otherwise one kernel per op, any dtype.
    ``recompute_activation``: ``act`` is not kept; backward rebuilds it from ``fc1`` for dW2.
    """

    @staticmethod
    def forward(ctx, x, w1, w2, group_list, group_list_type, probs, recompute_activation, fused_kernels,
                differentiated=True):
        if fused_kernels:
            fc1, act, gl, p = _gmm_swiglu_forward(x, w1, group_list, group_list_type, probs, want_fc1=differentiated)
        else:
            _lib.require_device(x, "x")
            gl = _group_list_tensor(group_list, x.device)
            fc1 = gmm_raw(x, w1, gl, 0, group_list_type)
            p = None
            if probs is not None:
                _lib.require_device(probs, "probs")
                p = probs.contiguous().view(-1)
                if p.numel() != fc1.size(0):
                    raise RuntimeError(f"probs has {p.numel()} entries, expected {fc1.size(0)}")
            if fc1.size(1) % 2 != 0:
                raise RuntimeError(f"the first matmul must produce an even number of columns, got {fc1.size(1)}")
            act = _swiglu_from_fc1(fc1, p)
        if w2.dim() != 3 or w2.size(0) != w1.size(0) or w2.size(1) != act.size(1) or w2.dtype != x.dtype:
            raise ValueError(f"w2 {tuple(w2.shape)} {w2.dtype} does not match the activation {tuple(act.shape)} {act.dtype}")
        out = gmm_raw(act, w2, gl, 0, group_list_type)
        if differentiated:
            ctx.save_for_backward(x, w1, w2, gl, fc1, p, None if recompute_activation else act)
        ctx.group_list_type = group_list_type
        ctx.fused_kernels = fused_kernels
        ctx.probs_shape = None if probs is None else probs.shape
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w1, w2, gl, fc1, p, act = ctx.saved_tensors
        dev = grad_out.device
        glt = ctx.group_list_type
        dy = grad_out.contiguous()
        if act is None:
            act = _swiglu_from_fc1(fc1, p)
        # everything the side stream writes is allocated here, on the caller's stream
        dw1 = torch.empty(w1.shape, dtype=w1.dtype, device=dev) if ctx.needs_input_grad[1] else None
        dw2 = torch.empty(w2.shape, dtype=w2.dtype, device=dev) if ctx.needs_input_grad[2] else None
        side = _beside(dy)
        with side:                                   # dW2 needs only act and dy
            if dw2 is not None:
                gmm_raw(act.t(), dy, gl, 2, glt, out=dw2)
        if ctx.fused_kernels:
            d_fc1, gp = K.gmm_swiglu_grad(dy, w2.contiguous(), fc1, p, gl, glt)
            gp = gp if p is not None else None
        else:
            dact = gmm_raw(dy, w2.transpose(1, 2), gl, 0, glt)
            d_fc1, gp = _swiglu_grad_from_fc1(dact, fc1, p)
        with side.again():                           # dW1 needs d_fc1: the side stream picks up from here
            if dw1 is not None:
                gmm_raw(x.t(), d_fc1, gl, 2, glt, out=dw1)
        dx = gmm_raw(d_fc1, w1.transpose(1, 2), gl, 0, glt) if ctx.needs_input_grad[0] else None
        side.join()
        gp_out = gp.view(ctx.probs_shape) if (gp is not None and ctx.needs_input_grad[5]) else None
        return dx, dw1, dw2, None, None, gp_out, None, None, None


def grouped_mlp(x, w1, w2, group_list, probs=None, *, group_list_type: int = 1, recompute_activation: bool = False,
                fused_kernels: bool = True):
    """``gmm(silu(gate) * up * probs, w2)`` with ``gate | up = gmm(x, w1)``: the expert MLP as one autograd node.
    ``w1 [E, K, 2*ffn]``, ``w2 [E, ffn, K']``.  ``fused_kernels`` (default) fuses both SwiGLU passes into the
    neighbouring grouped matmuls and needs the layout conditions of :func:`gmm_swiglu`; without it every op is
    its own kernel, for any dtype and layout the grouped matmul takes."""
    return GroupedMLPFunction.apply(x, w1, w2, group_list, group_list_type, probs, recompute_activation, fused_kernels,
                                    _differentiated(x, w1, w2, probs))
