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

__all__ = ["sort_chunks_by_idxs"]


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
