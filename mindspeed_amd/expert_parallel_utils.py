"""``permute`` / ``unpermute`` of the expert-parallel dispatcher, index form.

Mirrors mindspeed/fsdp/distributed/expert_parallel/utils.py:10-69 (twin: mindspeed/lite/distributed/
expert_parallel/utils.py:6-41).  ``fused_permute`` / ``fused_unpermute`` are the calls ``dispatch_mlp_combine(fused=True)``
makes (there through the ``torch_npu`` namespace, here on ``npu_moe_token_permute`` / ``npu_moe_token_unpermute``):
the second value of ``fused_permute`` is the int32 row map the fused unpermute consumes.  With ``fused=False`` the
reference runs plain torch ops and its second value is the forward order ``stable_argsort(indices)`` in the indices'
dtype; the same convention is served here by the same kernels (the permute kernel emits that order as a by-product,
and the unpermute inverts it on the device), since this package has no torch path.
"""
from __future__ import annotations

import torch

from .ops import moe_token_permute_with_aux, npu_moe_token_permute, npu_moe_token_unpermute
from .ops._kernels import K

__all__ = ["permute", "unpermute", "fused_permute", "fused_unpermute", "eager_permute", "eager_unpermute",
           "normalize_expert_args"]


def fused_permute(tokens, indices):
    return npu_moe_token_permute(tokens, indices)


def eager_permute(tokens, indices):
    """``(tokens.index_select(0, sorted_indices // topk), sorted_indices)`` with ``sorted_indices =
    argsort(indices.view(-1), stable=True)`` in the dtype of ``indices`` (utils.py:10-15)."""
    permuted, _row_id_map, sorted_indices, _ = moe_token_permute_with_aux(tokens, indices)
    return permuted, sorted_indices.to(indices.dtype)


def permute(tokens, indices, fused=False):
    return fused_permute(tokens, indices) if fused else eager_permute(tokens, indices)


def fused_unpermute(permuted_tokens, sorted_indices, probs):
    if probs is not None:
        permuted_tokens = permuted_tokens.to(probs.dtype)      # utils.py:37-38
    return npu_moe_token_unpermute(permuted_tokens, sorted_indices, probs)


def eager_unpermute(permuted_tokens, sorted_indices, probs):
    """``sorted_indices`` in the forward order of :func:`eager_permute` (row ``r`` came from flat position
    ``sorted_indices[r]``): ``out[t] = sum_j probs[t, j] * permuted_tokens[row of position t * topk + j]``
    (utils.py:26-34).  Every flat position must own a row (the reference's ``index_copy_`` has no dropped rows
    either)."""
    num_flat = permuted_tokens.size(0) if probs is None else probs.numel()
    if sorted_indices.numel() != num_flat:
        raise RuntimeError(f"sorted_indices has {sorted_indices.numel()} entries, expected one per (token, slot) pair: "
                           f"{num_flat}")
    order = sorted_indices.reshape(-1).to(torch.int32).contiguous()
    # row_id_map[sorted_indices[r]] = r: the positions 0..n-1 scattered by the forward order (bit copies of int32
    # values moved as 4-byte elements)
    rows = torch.arange(num_flat, dtype=torch.int32, device=order.device).view(torch.float32)
    row_id_map = K.move_rows(rows, order, True, False).view(torch.int32)
    return npu_moe_token_unpermute(permuted_tokens, row_id_map, probs)


def unpermute(permuted_tokens, sorted_indices, probs=None, fused=False):
    if permuted_tokens.size(0) != sorted_indices.numel():
        raise AssertionError(f'permuted tokens({permuted_tokens.size(0)}) != sorted indices({sorted_indices.size()})')
    return fused_unpermute(permuted_tokens, sorted_indices, probs) if fused \
        else eager_unpermute(permuted_tokens, sorted_indices, probs)


def normalize_expert_args(top_k_index, top_k_weights):
    """``(indices, weights)`` whichever way round they were passed, the weights gathered to the indices' shape if they
    came as a full ``[tokens, experts]`` matrix (utils.py:49-69)."""
    if torch.is_floating_point(top_k_index):
        top_k_index, top_k_weights = top_k_weights, top_k_index
    if top_k_weights.size() != top_k_index.size():
        top_k_weights = top_k_weights.gather(1, top_k_index)
    return top_k_index, top_k_weights
