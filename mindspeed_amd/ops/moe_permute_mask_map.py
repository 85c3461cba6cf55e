"""Routing-map (mask) mode of MoE permute / unpermute on MI355X.

Mirrors ``permute`` / ``unpermute`` of mindspeed/core/fusions/fused_moe_permute.py:50-85 and the
autograd Functions ``MoePermuteMaskMap`` / ``MoeUnpermuteMaskMap`` of
mindspeed/te/pytorch/permutation.py:12-148, which wrap the vendor ops
``torch_npu.npu_moe_token_permute_with_routing_map[_grad]`` and
``torch_npu._npu_moe_token_unpermute_with_routing_map[_grad]``.  Those follow Megatron-LM core_r0.12
``megatron/core/transformer/moe/moe_utils.py`` ``permute`` / ``unpermute`` (the reference's
``fused=False`` branch calls them directly, fused_moe_permute.py:65-66,84-85):

* ``routing_map`` is a ``[num_tokens, num_experts]`` bool mask, ``probs`` a same-shaped matrix;
* rows come out expert-major, token-ascending: ``sorted_indices`` (int64 token ids) is
  ``arange(T).expand(E, T).masked_select(routing_map.T)``, ``permuted_probs`` is
  ``probs.T.masked_select(routing_map.T)`` (the in-tree restatement is
  mindspeed/core/transformer/moe/moe_feature/overlap/token_dispatcher.py:451-453);
* with ``drop_and_pad`` every expert gets ``capacity = num_out_tokens // num_experts`` rows:
  ``routing_map.T.argsort(descending, stable)[:, :capacity]``, i.e. its routed tokens first and
  non-routed tokens as padding;
* unpermute is ``zeros(restore_shape).scatter_add_(0, sorted_indices, permuted * permuted_probs)``
  (in-tree restatement: mindspeed/core/transformer/moe/unpermute_without_activation.py:35-68).

Here both directions run the HIP kernels of the index form with ``topk = num_experts``: the mask is
turned into sort keys on the device and the resulting row map drives the same row movers.  The ``fused``
flag is accepted for signature compatibility; there is no second code path.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .. import _lib, flop_counter

__all__ = ["permute", "unpermute", "MoePermuteMaskMap", "MoeUnpermuteMaskMap", "routing_map_row_maps"]


def _check_map(routing_map, num_tokens=None):
    if routing_map is None:
        raise ValueError("routing_map is required")
    if routing_map.dim() != 2:
        raise RuntimeError(f"routing_map should be 2 dimensional, but got {routing_map.dim()}-dimensional.")
    if routing_map.dtype != torch.bool:
        raise TypeError(f"routing_map dtype [{routing_map.dtype}] is invalid, should be bool")
    _lib.require_device(routing_map, "routing_map")
    if num_tokens is not None and routing_map.size(0) != num_tokens:
        raise RuntimeError(f"routing_map has {routing_map.size(0)} rows, expected {num_tokens}")


def routing_map_row_maps(routing_map: torch.Tensor, num_rows: int, drop_and_pad: bool = False,
                         tokens: Optional[torch.Tensor] = None, want_counts: bool = False):
    """Sort the mask on the device.

    Returns ``(permuted_tokens or None, row_id_map, sorted_flat, tokens_per_expert or None)``:
    ``row_id_map`` (int32 ``[T*E]``) is the output row of flat entry ``t*E+e`` (dropped entries hold
    ``0x7fffffff``), ``sorted_flat`` (int32 ``[num_rows]``) its inverse.  With ``tokens`` the rows are
    moved in the same call.
    """
    lib = _lib.load()
    _check_map(routing_map)
    routing_map = routing_map.contiguous()
    num_tokens, num_experts = routing_map.shape
    num_rows = int(num_rows)
    dev = routing_map.device
    if drop_and_pad and (num_rows % num_experts != 0 or num_rows // num_experts > num_tokens):
        raise RuntimeError(f"drop_and_pad needs num_out_tokens = num_experts * capacity with capacity <= num_tokens, "
                           f"got {num_rows} for {num_experts} experts and {num_tokens} tokens")
    if not 0 <= num_rows <= num_tokens * num_experts:
        raise RuntimeError(f"num_out_tokens {num_rows} outside [0, {num_tokens * num_experts}]")
    row_id_map = torch.empty(num_tokens * num_experts, dtype=torch.int32, device=dev)
    sorted_flat = torch.empty(num_rows, dtype=torch.int32, device=dev)
    counts = torch.empty(num_experts, dtype=torch.int64, device=dev) if want_counts else None
    permuted = None
    hidden, dtype_code, elem = 1, _lib.dtype_code(torch.float32, "tokens"), 0
    if tokens is not None:
        tokens = tokens.contiguous()
        hidden = tokens.size(1)
        if hidden == 0:
            raise RuntimeError("tokens must have a non-empty hidden dimension")
        dtype_code = _lib.dtype_code(tokens.dtype, "tokens")
        elem = tokens.element_size()
        permuted = torch.empty((num_rows, hidden), dtype=tokens.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_moe_routing_map_workspace_size(num_tokens, num_experts, int(bool(drop_and_pad)),
                                                     ctypes.byref(nbytes)), "ms_moe_routing_map_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    work = (num_tokens * hidden * elem + num_rows * hidden * elem if tokens is not None else 0) \
        + num_tokens * num_experts * (1 + 4) + num_rows * 4
    with torch.cuda.device(dev), flop_counter.op("permute", work, "byte", dev):
        _lib.check(lib.ms_moe_routing_map_permute(
            _lib.stream_ptr(dev), _lib.ptr(tokens), _lib.ptr(routing_map), num_tokens, num_experts, hidden, dtype_code,
            num_rows, int(bool(drop_and_pad)), _lib.ptr(permuted), _lib.ptr(row_id_map), _lib.ptr(sorted_flat),
            _lib.ptr(counts), _lib.ptr(ws), ws.numel()), "ms_moe_routing_map_permute")
    return permuted, row_id_map, sorted_flat, counts


# The dispatcher hands the ``sorted_indices`` it got from ``permute`` back to ``unpermute`` together with the
# same ``routing_map``.  The row map that ``permute`` computed from that mask travels along on the tensor, so
# ``unpermute`` does not have to sort the mask again; it is only used when the mask is still the same tensor
# in the same state (same storage, shape and version counter) and the row count and mode match.
def _map_key(routing_map, num_rows, drop_and_pad):
    return (routing_map.data_ptr(), tuple(routing_map.shape), routing_map._version, int(num_rows), bool(drop_and_pad))


def _remember_row_map(sorted_indices, routing_map, row_id_map, drop_and_pad):
    sorted_indices._ms_row_map = (_map_key(routing_map, sorted_indices.numel(), drop_and_pad), row_id_map)


def _recall_row_map(sorted_indices, routing_map, num_rows, drop_and_pad):
    cached = getattr(sorted_indices, "_ms_row_map", None)
    if cached is not None and cached[0] == _map_key(routing_map, num_rows, drop_and_pad):
        return cached[1]
    return None


def _resolve_num_rows(routing_map, num_out_tokens, drop_and_pad):
    if drop_and_pad:
        if num_out_tokens is None:
            raise ValueError("drop_and_pad needs num_out_tokens (= num_experts * capacity)")
        num_experts = routing_map.size(1)
        return (int(num_out_tokens) // num_experts) * num_experts   # capacity = num_out_tokens // num_experts
    if num_out_tokens is None:
        # masked_select in the torch path reads the count back to the host as well
        return int(routing_map.sum().item())
    return int(num_out_tokens)


class MoePermuteMaskMap(torch.autograd.Function):
    """functional Permute with mask router map (mindspeed/te/pytorch/permutation.py:12-65)"""

    @staticmethod
    def forward(ctx, tokens, routing_map, probs: Optional[torch.Tensor] = None,
                num_out_tokens: Optional[int] = None, drop_and_pad: bool = False
                ) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
        if tokens.dim() != 2:
            raise RuntimeError(f"The dims of input tokens should be 2 dimensional, but got {tokens.dim()}-dimensional.")
        if routing_map is not None and routing_map.dtype != torch.bool:
            raise TypeError(f"routing_map dtype [{routing_map.dtype}] is invalid, should be bool")
        _lib.require_device(tokens, "tokens")
        _check_map(routing_map, tokens.size(0))
        lib = _lib.load()
        num_tokens, num_experts = routing_map.shape
        num_rows = _resolve_num_rows(routing_map, num_out_tokens, drop_and_pad)
        permuted, row_id_map, sorted_flat, _ = routing_map_row_maps(routing_map, num_rows, drop_and_pad, tokens)
        dev = tokens.device
        permuted_probs = None
        if probs is not None:
            _lib.require_device(probs, "probs")
            if probs.shape != routing_map.shape:
                raise RuntimeError(f"probs shape {tuple(probs.shape)} differs from routing_map shape "
                                   f"{tuple(routing_map.shape)}")
            probs = probs.contiguous()
            permuted_probs = torch.empty(num_rows, dtype=probs.dtype, device=dev)
        sorted_indices = torch.empty(num_rows, dtype=torch.int64, device=dev)
        with torch.cuda.device(dev):
            _lib.check(lib.ms_moe_routing_map_probs(
                _lib.stream_ptr(dev), _lib.ptr(sorted_flat), num_rows, num_experts, _lib.ptr(probs),
                _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0, _lib.ptr(permuted_probs),
                _lib.ptr(sorted_indices)), "ms_moe_routing_map_probs")
        ctx.save_for_backward(row_id_map)
        ctx.set_materialize_grads(False)
        ctx.num_tokens = num_tokens
        ctx.num_experts = num_experts
        ctx.num_rows = num_rows
        ctx.probs_dtype = probs.dtype if probs is not None else None
        ctx.mark_non_differentiable(sorted_indices)
        _remember_row_map(sorted_indices, routing_map, row_id_map, drop_and_pad)
        return permuted, permuted_probs, sorted_indices

    @staticmethod
    def backward(ctx, permuted_act_grad, permuted_probs_grad, _):
        (row_id_map,) = ctx.saved_tensors
        lib = _lib.load()
        act_grad = None
        probs_grad = None
        if ctx.needs_input_grad[0] and permuted_act_grad is not None:
            permuted_act_grad = permuted_act_grad.contiguous()
            dev = permuted_act_grad.device
            hidden = permuted_act_grad.size(1)
            act_grad = torch.empty((ctx.num_tokens, hidden), dtype=permuted_act_grad.dtype, device=dev)
            work = flop_counter.permute_grad_bytes(ctx.num_tokens, ctx.num_experts, hidden,
                                                   permuted_act_grad.element_size(), ctx.num_rows)
            with torch.cuda.device(dev), flop_counter.op("permute_grad", work, "byte", dev):
                _lib.check(lib.ms_moe_token_permute_grad(
                    _lib.stream_ptr(dev), _lib.ptr(permuted_act_grad), _lib.ptr(row_id_map), ctx.num_tokens,
                    ctx.num_experts, hidden, _lib.dtype_code(permuted_act_grad.dtype, "permuted_act_grad"),
                    ctx.num_rows, _lib.ptr(act_grad)), "ms_moe_token_permute_grad")
        if ctx.needs_input_grad[2] and permuted_probs_grad is not None:
            permuted_probs_grad = permuted_probs_grad.contiguous().to(ctx.probs_dtype)
            dev = permuted_probs_grad.device
            probs_grad = torch.empty((ctx.num_tokens, ctx.num_experts), dtype=ctx.probs_dtype, device=dev)
            with torch.cuda.device(dev):
                _lib.check(lib.ms_moe_routing_map_probs_grad(
                    _lib.stream_ptr(dev), _lib.ptr(row_id_map), row_id_map.numel(), _lib.ptr(permuted_probs_grad),
                    _lib.dtype_code(ctx.probs_dtype, "probs"), ctx.num_rows, _lib.ptr(probs_grad)),
                    "ms_moe_routing_map_probs_grad")
        return act_grad, None, probs_grad, None, None


class MoeUnpermuteMaskMap(torch.autograd.Function):
    """functional Unpermute with mask router map (mindspeed/te/pytorch/permutation.py:68-148)"""

    @staticmethod
    def forward(ctx, permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, restore_shape: torch.Size,
                probs: Optional[torch.Tensor] = None, routing_map: Optional[torch.Tensor] = None,
                drop_and_pad: bool = False) -> torch.Tensor:
        if not permuted_tokens.numel():   # permutation.py:81-83
            ctx.empty = True
            ctx.probs = probs
            return permuted_tokens
        ctx.empty = False
        if permuted_tokens.dim() != 2:
            raise RuntimeError("The dims of input permuted_tokens should be 2 dimensional, "
                               f"but got {permuted_tokens.dim()}-dimensional.")
        if routing_map is None:
            raise ValueError("routing_map is required")
        _lib.require_device(permuted_tokens, "permuted_tokens")
        if sorted_indices.numel() != permuted_tokens.size(0):   # unpermute_without_activation.py:35-36
            raise AssertionError("sorted_indices must have one entry per permuted row")
        num_tokens = int(restore_shape[0])
        _check_map(routing_map, num_tokens)
        lib = _lib.load()
        permuted_tokens = permuted_tokens.contiguous()
        num_experts = routing_map.size(1)
        num_rows, hidden = permuted_tokens.shape
        row_id_map = _recall_row_map(sorted_indices, routing_map, num_rows, drop_and_pad)
        if row_id_map is None:
            _, row_id_map, _, _ = routing_map_row_maps(routing_map, num_rows, drop_and_pad)
        dev = permuted_tokens.device
        if probs is not None:
            _lib.require_device(probs, "probs")
            if probs.shape != routing_map.shape:
                raise RuntimeError(f"probs shape {tuple(probs.shape)} differs from routing_map shape "
                                   f"{tuple(routing_map.shape)}")
            ctx.probs_dtype = probs.dtype
            probs = probs.contiguous().to(permuted_tokens.dtype)
        out = torch.empty((num_tokens, hidden), dtype=permuted_tokens.dtype, device=dev)
        work = flop_counter.unpermute_bytes(num_tokens, num_experts, hidden, permuted_tokens.element_size(), num_rows)
        with torch.cuda.device(dev), flop_counter.op("unpermute", work, "byte", dev):
            _lib.check(lib.ms_moe_token_unpermute(
                _lib.stream_ptr(dev), _lib.ptr(permuted_tokens), _lib.ptr(row_id_map), _lib.ptr(probs), num_tokens,
                num_experts, hidden, _lib.dtype_code(permuted_tokens.dtype, "permuted_tokens"), num_rows,
                _lib.ptr(out)), "ms_moe_token_unpermute")
        ctx.save_for_backward(permuted_tokens if probs is not None else None, row_id_map, probs)
        ctx.num_tokens, ctx.num_experts, ctx.num_rows, ctx.hidden = num_tokens, num_experts, num_rows, hidden
        return out

    @staticmethod
    def backward(ctx, unpermuted_tokens_grad):
        if ctx.empty:   # permutation.py:104-105
            return unpermuted_tokens_grad, None, None, ctx.probs, None, None
        permuted_tokens, row_id_map, probs = ctx.saved_tensors
        lib = _lib.load()
        grad_out = unpermuted_tokens_grad.contiguous()
        dev = grad_out.device
        # every row has exactly one entry mapping to it (rows nothing maps to exist only when the caller's
        # row count exceeds the number of mapped entries; they belong to no expert and stay unwritten)
        grad_permuted = torch.empty((ctx.num_rows, ctx.hidden), dtype=grad_out.dtype, device=dev)
        grad_probs = torch.empty_like(probs) if probs is not None else None
        work = flop_counter.unpermute_grad_bytes(ctx.num_tokens, ctx.num_experts, ctx.hidden, grad_out.element_size(),
                                                 ctx.num_rows, probs is not None)
        with torch.cuda.device(dev), flop_counter.op("unpermute_grad", work, "byte", dev):
            _lib.check(lib.ms_moe_token_unpermute_grad(
                _lib.stream_ptr(dev), _lib.ptr(permuted_tokens), _lib.ptr(grad_out), _lib.ptr(row_id_map),
                _lib.ptr(probs), ctx.num_tokens, ctx.num_experts, ctx.hidden,
                _lib.dtype_code(grad_out.dtype, "unpermuted_tokens_grad"), ctx.num_rows, _lib.ptr(grad_permuted),
                _lib.ptr(grad_probs)), "ms_moe_token_unpermute_grad")
        if grad_probs is not None:
            grad_probs = grad_probs.to(ctx.probs_dtype)
            if not ctx.needs_input_grad[3]:
                grad_probs = None
        return grad_permuted, None, None, grad_probs, None, None


def permute(tokens, routing_map, probs: Optional[torch.Tensor] = None, num_out_tokens: Optional[int] = None,
            fused: bool = False, drop_and_pad: bool = False):
    """``(permuted_tokens, permuted_probs, sorted_indices)`` for a bool ``routing_map`` ``[T, E]``.

    Without ``num_out_tokens`` the number of set entries is read back to the host (as ``masked_select``
    does in the torch path); with it, it must equal that number (rows past it are left unwritten and
    belong to no expert).  With ``drop_and_pad`` it is ``num_experts * capacity``.
    """
    return MoePermuteMaskMap.apply(tokens, routing_map, probs, num_out_tokens, drop_and_pad)


def unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, restore_shape: torch.Size,
              probs: torch.Tensor = None, routing_map: torch.Tensor = None, fused: bool = False,
              drop_and_pad: bool = False) -> torch.Tensor:
    """``out[t] = sum_e probs[t, e] * permuted_tokens[row of (t, e)]`` over the mapped entries of token ``t``
    (weights 1 without ``probs``); fp32 accumulation, one rounding.  ``routing_map`` is required: the row
    of an entry is recomputed from it on the device."""
    return MoeUnpermuteMaskMap.apply(permuted_tokens, sorted_indices, restore_shape, probs, routing_map, drop_and_pad)
