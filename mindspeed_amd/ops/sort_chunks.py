"""``sort_chunks_by_idxs`` on MI355X.

Mirrors the dispatcher hook restated in mindspeed/core/transformer/moe/
moe_feature/overlap/moe_common.py:377-398 (fused form:
mindspeed/lite/ops/triton/sort_chunks_by_idx.py:300-348):
``cat([split(input, split_sizes)[i] for i in sorted_idxs])``; the backward is
the inverse row map.  ``split_sizes`` and ``sorted_idxs`` may be device
tensors; nothing is read back to the host.  Given as host lists they are checked
(``sorted_idxs`` a permutation, the sizes summing to the row count, which the
reference's ``split`` / ``cat`` require too); device tensors cannot be checked
without a read-back, so then the outputs and gradients are zero-initialised and
rows that a partial map leaves out read as zeros.
"""
from __future__ import annotations

import torch

from .. import _lib
from ._kernels import K

__all__ = ["sort_chunks_by_idxs", "moe_sort_chunks_by_index", "moe_sort_chunks_by_index_with_probs",
           "make_chunk_sort_map", "sort_chunks_by_map"]


def _as_i64(v, device):
    if isinstance(v, torch.Tensor):
        return v.to(device=device, dtype=torch.int64).contiguous()
    return torch.tensor(list(v), dtype=torch.int64, device=device)


class _SortChunks(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, split_sizes, sorted_idxs, probs, checked):
        ctx.checked = checked
        _lib.require_device(inp, "input")
        if inp.dim() != 2:
            raise RuntimeError(f"input must be 2 dimensional, got {inp.dim()}-dimensional")
        inp = inp.contiguous()
        rows = inp.size(0)
        p = probs.contiguous() if probs is not None else None
        if p is not None and p.numel() != rows:
            raise RuntimeError(f"probs has {p.numel()} entries, expected {rows}")
        out, out_p, row_map = K.sort_chunks(inp, split_sizes, sorted_idxs, p, not checked)
        ctx.save_for_backward(row_map)
        ctx.set_materialize_grads(False)
        ctx.has_probs = p is not None
        ctx.mark_non_differentiable(row_map)
        if p is None:
            return out, None, row_map
        return out, out_p, row_map

    @staticmethod
    def backward(ctx, grad_out, grad_probs, _grad_map):
        (row_map,) = ctx.saved_tensors
        if grad_out is None:
            return None, None, None, None, None
        gi = K.gather_rows(grad_out.contiguous(), row_map, not ctx.checked)
        gp = None
        if ctx.has_probs and grad_probs is not None:
            gp = K.gather_rows(grad_probs.contiguous(), row_map, not ctx.checked)
        return gi, None, None, gp, None


def sort_chunks_by_idxs(input, split_sizes, sorted_idxs, probs=None, fused=True):
    """Returns ``(output, permuted_probs)`` like the reference hook."""
    del fused  # one code path
    dev = input.device
    on_host = lambda v: not isinstance(v, torch.Tensor) or v.device.type == "cpu"     # noqa: E731
    checked = on_host(split_sizes) and on_host(sorted_idxs)
    if checked:
        as_list = lambda v: [int(i) for i in (v.tolist() if isinstance(v, torch.Tensor) else v)]     # noqa: E731
        sizes, order = as_list(split_sizes), as_list(sorted_idxs)
        if sorted(order) != list(range(len(sizes))):
            raise RuntimeError(f"sorted_idxs must be a permutation of 0..{len(sizes) - 1}, got {order}")
        if min(sizes, default=0) < 0 or sum(sizes) != input.size(0):
            raise RuntimeError(f"split_sizes {sizes} do not sum to the {input.size(0)} rows of input")
    split_sizes = _as_i64(split_sizes, dev)
    sorted_idxs = _as_i64(sorted_idxs, dev)
    if split_sizes.numel() != sorted_idxs.numel():
        raise RuntimeError("split_sizes and sorted_idxs must have the same length")
    out, out_probs, _ = _SortChunks.apply(input, split_sizes, sorted_idxs, probs, checked)
    return out, out_probs


# ---- the fused form's own names (mindspeed/lite/ops/triton/sort_chunks_by_idx.py) ------------------------------------
def make_chunk_sort_map(split_sizes: torch.Tensor, sorted_indices: torch.Tensor, num_tokens: int, num_splits: int):
    """``row_id_map`` int32 ``[num_tokens]``: entry ``r`` is the output row of source row ``r``
    (sort_chunks_by_idx.py:67-115).  Rows past the sum of ``split_sizes`` map to -1."""
    _lib.require_device(split_sizes, "split_sizes")
    _lib.require_device(sorted_indices, "sorted_indices")
    if split_sizes.numel() != num_splits or sorted_indices.numel() != num_splits:
        raise AssertionError("sorted_idxs size is not equal to num_splits.")
    dev = split_sizes.device
    return K.chunk_sort_map(_as_i64(split_sizes, dev), _as_i64(sorted_indices, dev), int(num_tokens))


def sort_chunks_by_map(inp: torch.Tensor, row_id_map: torch.Tensor, probs, num_tokens: int, hidden_size: int,
                       is_forward: bool):
    """Move rows (and optionally one probability per row) by a map from :func:`make_chunk_sort_map`: forward
    ``out[row_id_map[i]] = inp[i]``, backward ``out[i] = inp[row_id_map[i]]`` (sort_chunks_by_idx.py:118-221).
    Returns ``(output, permuted_probs or None)``."""
    _lib.require_device(inp, "input")
    if inp.dim() != 2 or inp.size(0) != num_tokens or inp.size(1) != hidden_size:
        raise RuntimeError(f"input must be [{num_tokens}, {hidden_size}], got {tuple(inp.shape)}")
    if row_id_map.dtype != torch.int32 or row_id_map.numel() != num_tokens:
        raise RuntimeError("row_id_map must hold one int32 entry per row")
    out = K.move_rows(inp.contiguous(), row_id_map, bool(is_forward), False)
    out_probs = None
    if probs is not None:
        if probs.numel() != num_tokens:
            raise RuntimeError(f"probs has {probs.numel()} entries, expected {num_tokens}")
        out_probs = K.move_rows(probs.contiguous().view(-1), row_id_map, bool(is_forward), False)
    return out, out_probs


def _check_fused_args(inp, split_sizes, sorted_index, probs):
    # sort_chunks_by_idx.py:238-252: the fused form takes device tensors only
    for name, t in (("inp", inp), ("split_sizes", split_sizes), ("sorted_idxs", sorted_index), ("probs", probs)):
        if t is not None and (not isinstance(t, torch.Tensor) or t.device.type not in ("cuda", "meta")):
            raise AssertionError(f"This operation needs {name} on the device")
    if split_sizes.size(0) != sorted_index.size(0):
        raise AssertionError("sorted_idxs size is not equal to num_splits.")


def moe_sort_chunks_by_index(inp: torch.Tensor, split_sizes: torch.Tensor, sorted_index: torch.Tensor):
    """``cat([split(inp, split_sizes)[i] for i in sorted_index])`` (sort_chunks_by_idx.py:300-318); differentiable
    w.r.t. ``inp``.  One launch: the map and the row movement come from the same kernel."""
    if not inp.numel():
        return inp
    _check_fused_args(inp, split_sizes, sorted_index, None)
    out, _ = sort_chunks_by_idxs(inp, split_sizes, sorted_index, None)
    return out


def moe_sort_chunks_by_index_with_probs(inp: torch.Tensor, probs: torch.Tensor, split_sizes: torch.Tensor,
                                        sorted_index: torch.Tensor):
    """The same with one probability per row moved along (sort_chunks_by_idx.py:321-348); differentiable w.r.t.
    ``inp`` and ``probs``."""
    if not inp.numel():
        return inp, probs
    _check_fused_args(inp, split_sizes, sorted_index, probs)
    return sort_chunks_by_idxs(inp, split_sizes, sorted_index, probs)
