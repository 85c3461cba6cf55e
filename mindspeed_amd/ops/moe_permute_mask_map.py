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
turned into sort keys on the device and the resulting row map drives the same row movers.  There is no second
code path: ``fused`` only selects the reference hook's dtype rule for mixed fp32 / 16-bit operands (see
:func:`permute`).
"""
from __future__ import annotations

from typing import Optional, Tuple

import os
import weakref

import torch

from .. import _lib
from ._kernels import K

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
    _check_map(routing_map)
    routing_map = routing_map.contiguous()
    num_tokens, num_experts = routing_map.shape
    num_rows = int(num_rows)
    if drop_and_pad and (num_rows % num_experts != 0 or num_rows // num_experts > num_tokens):
        raise RuntimeError(f"drop_and_pad needs num_out_tokens = num_experts * capacity with capacity <= num_tokens, "
                           f"got {num_rows} for {num_experts} experts and {num_tokens} tokens")
    if not 0 <= num_rows <= num_tokens * num_experts:
        raise RuntimeError(f"num_out_tokens {num_rows} outside [0, {num_tokens * num_experts}]")
    if tokens is not None:
        tokens = tokens.contiguous()
        if tokens.size(1) == 0:
            raise RuntimeError("tokens must have a non-empty hidden dimension")
        _lib.dtype_code(tokens.dtype, "tokens")
    permuted, row_id_map, sorted_flat, counts = K.routing_map_permute(
        tokens, routing_map, num_rows, bool(drop_and_pad), bool(want_counts))
    return (permuted if tokens is not None else None), row_id_map, sorted_flat, (counts if want_counts else None)


# The dispatcher hands ``unpermute`` the same ``routing_map`` tensor it gave ``permute``.  The row maps that
# ``permute`` computed from that mask are remembered on the mask tensor itself, so ``unpermute`` need not sort the mask
# again whatever happened to ``sorted_indices`` in between (clones, views, an exchange between ranks).  They are only
# used while the mask is that same tensor object in the same state — version counter, storage address and shape — and
# the row count and mode match; any other mask, a view or a copy of it included, is sorted afresh.  A write that
# bypasses the version counter (``routing_map.data.copy_()``, ``set_()`` onto the same address, a write through a
# DLPack / numpy alias) is not seen: a mask changed that way must be permuted again before it is unpermuted, or the
# memory switched off with ``MINDSPEED_AMD_ROW_MAP_CACHE=0``.  A map reused on another stream than the one that
# produced it first waits for that stream.
_ROW_MAPS_KEPT = 4
_ROW_MAP_CACHE = os.environ.get("MINDSPEED_AMD_ROW_MAP_CACHE", "1") != "0"
_CHECK_SORTED_INDICES = os.environ.get("MINDSPEED_AMD_CHECK_SORTED_INDICES", "1") != "0"


def _mask_state(routing_map):
    return (routing_map._version, routing_map.data_ptr(), tuple(routing_map.shape), tuple(routing_map.stride()))


def _remember_row_map(routing_map, num_rows, drop_and_pad, row_id_map, sorted_flat, sorted_indices=None):
    if not _ROW_MAP_CACHE or _tracing(routing_map):
        return
    kept = getattr(routing_map, "_ms_row_maps", None)
    state = _mask_state(routing_map)
    if kept is None or kept[0] != state:
        kept = (state, {})
        routing_map._ms_row_maps = kept
    maps = kept[1]
    # (the last element: index tensors known to agree with the map, as weak references with their version counters)
    known = [] if sorted_indices is None else [(weakref.ref(sorted_indices), sorted_indices._version)]
    maps[(int(num_rows), bool(drop_and_pad))] = (row_id_map, sorted_flat, torch.cuda.current_stream(routing_map.device),
                                                 known)
    while len(maps) > _ROW_MAPS_KEPT:
        maps.pop(next(iter(maps)))


def _recall_row_map(routing_map, num_rows, drop_and_pad):
    """``(row_id_map, sorted_flat, known index tensors)`` of an earlier ``permute`` of this very mask, or None."""
    kept = getattr(routing_map, "_ms_row_maps", None)
    if not _ROW_MAP_CACHE or kept is None or kept[0] != _mask_state(routing_map):
        return None
    hit = kept[1].get((int(num_rows), bool(drop_and_pad)))
    if hit is None:
        return None
    row_id_map, sorted_flat, stream, known = hit
    now = torch.cuda.current_stream(routing_map.device)
    if now != stream:
        now.wait_stream(stream)          # everything queued on the producing stream so far, the map's kernel included
    return row_id_map, sorted_flat, known


def _is_known(known, sorted_indices) -> bool:
    for ref, version in known:
        if ref() is sorted_indices and version == sorted_indices._version:
            return True
    return False


def _tracing(t):
    return t.device.type == "meta" or torch.compiler.is_compiling() or \
        isinstance(t, torch._subclasses.fake_tensor.FakeTensor)


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
        num_tokens, num_experts = routing_map.shape
        num_rows = _resolve_num_rows(routing_map, num_out_tokens, drop_and_pad)
        permuted, row_id_map, sorted_flat, _ = routing_map_row_maps(routing_map, num_rows, drop_and_pad, tokens)
        if probs is not None:
            _lib.require_device(probs, "probs")
            if probs.shape != routing_map.shape:
                raise RuntimeError(f"probs shape {tuple(probs.shape)} differs from routing_map shape "
                                   f"{tuple(routing_map.shape)}")
            _lib.dtype_code(probs.dtype, "probs")
            probs = probs.contiguous()
        permuted_probs, sorted_indices = K.routing_map_probs(sorted_flat, probs, num_experts)
        if probs is None:
            permuted_probs = None
        ctx.save_for_backward(row_id_map)
        ctx.set_materialize_grads(False)
        ctx.num_tokens = num_tokens
        ctx.num_experts = num_experts
        ctx.num_rows = num_rows
        ctx.probs_dtype = probs.dtype if probs is not None else None
        ctx.mark_non_differentiable(sorted_indices)
        _remember_row_map(routing_map, num_rows, drop_and_pad, row_id_map, sorted_flat, sorted_indices)
        return permuted, permuted_probs, sorted_indices

    @staticmethod
    def backward(ctx, permuted_act_grad, permuted_probs_grad, _):
        (row_id_map,) = ctx.saved_tensors
        act_grad = None
        probs_grad = None
        if ctx.needs_input_grad[0] and permuted_act_grad is not None:
            act_grad = K.moe_token_permute_grad(permuted_act_grad.contiguous(), row_id_map, ctx.num_tokens,
                                                ctx.num_experts)
        if ctx.needs_input_grad[2] and permuted_probs_grad is not None:
            probs_grad = K.routing_map_probs_grad(row_id_map, permuted_probs_grad.contiguous().to(ctx.probs_dtype),
                                                  ctx.num_tokens, ctx.num_experts)
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
        permuted_tokens = permuted_tokens.contiguous()
        num_experts = routing_map.size(1)
        num_rows, hidden = permuted_tokens.shape
        kept = _recall_row_map(routing_map, num_rows, drop_and_pad)
        if kept is None:
            _, row_id_map, sorted_flat, _ = routing_map_row_maps(routing_map, num_rows, drop_and_pad)
            _remember_row_map(routing_map, num_rows, drop_and_pad, row_id_map, sorted_flat)
            kept = _recall_row_map(routing_map, num_rows, drop_and_pad)
        known = kept[2] if kept is not None else []
        if kept is not None:
            row_id_map, sorted_flat = kept[0], kept[1]
        # The rows are gathered by the map that the mask gives.  ``sorted_indices`` must say the same: the torch path
        # scatters row r to token sorted_indices[r] (unpermute_without_activation.py:54-62), so a re-ordered index
        # would mean another result there.  The tensor that ``permute`` itself returned for this mask is known to
        # agree; any other one is compared on the device once (one read-back of a flag; a tensor that passed is
        # remembered beside the map) unless MINDSPEED_AMD_CHECK_SORTED_INDICES=0.
        if _CHECK_SORTED_INDICES and not _tracing(sorted_indices) and not _is_known(known, sorted_indices):
            expect = torch.div(sorted_flat.clamp(min=0), num_experts, rounding_mode="floor")
            same = (sorted_indices.reshape(-1).to(expect.dtype) == expect) | (sorted_flat < 0)
            if not bool(same.all()):
                raise ValueError("sorted_indices is not the token order that routing_map gives (row r of permuted_tokens "
                                 "belongs to the r-th set entry of routing_map in expert-major order): unpermute "
                                 "recomputes the rows from routing_map and would silently ignore another order")
            known.append((weakref.ref(sorted_indices), sorted_indices._version))
            del known[:-4]
        if probs is not None:
            _lib.require_device(probs, "probs")
            if probs.shape != routing_map.shape:
                raise RuntimeError(f"probs shape {tuple(probs.shape)} differs from routing_map shape "
                                   f"{tuple(routing_map.shape)}")
            _lib.dtype_code(probs.dtype, "probs")
            probs = probs.contiguous()          # used in their own dtype, e.g. fp32 beside bf16 tokens
        out = K.moe_token_unpermute(permuted_tokens, row_id_map, probs, num_tokens, num_experts)
        ctx.save_for_backward(permuted_tokens if probs is not None else None, row_id_map, probs, sorted_flat)
        ctx.num_tokens, ctx.num_experts, ctx.num_rows, ctx.hidden = num_tokens, num_experts, num_rows, hidden
        ctx.all_rows_mapped = bool(drop_and_pad)      # every expert's capacity rows are filled (with padding entries)
        return out

    @staticmethod
    def backward(ctx, unpermuted_tokens_grad):
        if ctx.empty:   # permutation.py:104-105
            return unpermuted_tokens_grad, None, None, ctx.probs, None, None
        permuted_tokens, row_id_map, probs, sorted_flat = ctx.saved_tensors
        grad_out = unpermuted_tokens_grad.contiguous()
        # Every mapped row has exactly one entry leading to it and is written by the gradient kernel.  Rows that
        # nothing maps to exist only when the caller's row count exceeds the number of set mask entries; they are
        # marked in sorted_flat and written as zeros (a launch whose workgroups all return at once when there are none).
        grad_permuted, grad_probs = K.moe_token_unpermute_grad(
            permuted_tokens if probs is not None else grad_out.new_empty(0), grad_out, row_id_map, probs,
            ctx.num_tokens, ctx.num_experts, ctx.num_rows)
        if not ctx.all_rows_mapped:
            K.zero_unmapped_rows(grad_permuted, sorted_flat)
        if probs is None or not ctx.needs_input_grad[3]:
            grad_probs = None
        return grad_permuted, None, None, grad_probs, None, None


def permute(tokens, routing_map, probs: Optional[torch.Tensor] = None, num_out_tokens: Optional[int] = None,
            fused: bool = False, drop_and_pad: bool = False):
    """``(permuted_tokens, permuted_probs, sorted_indices)`` for a bool ``routing_map`` ``[T, E]``.

    Without ``num_out_tokens`` the number of set entries is read back to the host (as ``masked_select``
    does in the torch path); with it, it must equal that number (rows past it are left unwritten and
    belong to no expert).  With ``drop_and_pad`` it is ``num_experts * capacity``.

    Result dtypes follow the reference hook (mindspeed/core/fusions/fused_moe_permute.py:17-47,58-63).  With
    ``fused`` and exactly one of ``tokens`` / ``probs`` in fp32, the reference promotes both to fp32, permutes,
    and casts *both* results to the dtype of the operand that was not fp32; without ``fused`` (Megatron's own
    ``permute``) every result keeps its operand's dtype.  Both settings run the same kernels here.  A row copy
    moves bits, so 16-bit tokens are permuted as they are (the promotion and the cast back would change
    nothing); fp32 tokens next to 16-bit probabilities are permuted in fp32 and rounded afterwards, as the
    reference does, so their gradient is summed in fp32.
    """
    mixed = (fused and isinstance(probs, torch.Tensor)
             and (tokens.dtype == torch.float32) != (probs.dtype == torch.float32))
    if not mixed:
        return MoePermuteMaskMap.apply(tokens, routing_map, probs, num_out_tokens, drop_and_pad)
    if tokens.dtype != torch.float32:          # 16-bit tokens, fp32 probabilities: both results in the tokens' dtype
        permuted, permuted_probs, sorted_indices = MoePermuteMaskMap.apply(
            tokens, routing_map, probs, num_out_tokens, drop_and_pad)
        return permuted, permuted_probs.to(tokens.dtype), sorted_indices
    low = probs.dtype                          # fp32 tokens, 16-bit probabilities: both results in the probs' dtype
    permuted, permuted_probs, sorted_indices = MoePermuteMaskMap.apply(
        tokens, routing_map, probs.to(torch.float32), num_out_tokens, drop_and_pad)
    return permuted.to(low), permuted_probs.to(low), sorted_indices


def unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, restore_shape: torch.Size,
              probs: torch.Tensor = None, routing_map: torch.Tensor = None, fused: bool = False,
              drop_and_pad: bool = False) -> torch.Tensor:
    """``out[t] = sum_e probs[t, e] * permuted_tokens[row of (t, e)]`` over the mapped entries of token ``t``
    (weights 1 without ``probs``); fp32 accumulation, one rounding.  ``routing_map`` is required: the row
    of an entry is recomputed from it on the device."""
    return MoeUnpermuteMaskMap.apply(permuted_tokens, sorted_indices, restore_shape, probs, routing_map, drop_and_pad)
