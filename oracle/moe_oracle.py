"""CPU oracle for the per-rank MoE expert path.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain torch on the CPU, what the reference's open
pure-PyTorch path computes for token permute, grouped matmul, SwiGLU and the
prob-weighted unpermute.  It is a checker: only the test-suite, the smoke
check and the CPU-baseline leg of the benchmark may import it.  Nothing in
``mindspeed_amd`` (the product) imports or calls it.

Every function names the reference lines (relative to the reference root) it
follows.  How each function is pinned (what independent check would fail on a
plausible mistake) is listed next to it; the pins live in
``tests/test_oracle_pins.py``.

Pin status
----------
permute / row_id_map          pinned: brute-force ``sorted`` on tiny inputs,
                              ``numpy.argsort(kind="stable")``, the C counting
                              sort in ``permute_index_oracle.c``, permutation /
                              monotonic / tie-order invariants, the worked
                              example of the permute semantics.
unpermute                     pinned: fp64 triple-loop brute force, identity
                              ``unpermute(permute(x), 1/k) == x``.
permute_backward,
unpermute_backward            pinned: autograd of the forward restatement and
                              ``torch.autograd.gradcheck`` in fp64.
grouped_matmul / gmm_split    pinned: ``torch.bmm`` for equal groups,
                              ``torch.mm`` for one group, integer-valued
                              inputs (exact in every dtype), the reference
                              test's shapes and group lists.
gmm_backward                  pinned: autograd through the split-matmul form.
groupmatmul_add_fp32          pinned: equals ``out + dw`` (the reference
                              test's own identity).
swiglu                        pinned: closed form ``x*sigmoid(x)*u`` in fp64.
sort_chunks_by_idxs           pinned: brute-force row map.
permute_routing_map /         pinned: brute-force Python loops over (expert, token)
unpermute_routing_map         pairs incl. drop-and-pad, equality with the index
                              form (permute / unpermute above) on maps built from
                              top-k indices, the in-tree formulas
                              (token_dispatcher.py:451-453,
                              unpermute_without_activation.py:44-62); backward =
                              autograd of these differentiable restatements.
                              The algorithm itself is Megatron-LM core_r0.12
                              ``moe_utils.permute/unpermute`` (a dependency that
                              is not vendored in the reference tree), restated
                              from its published source.
fused_permute_routing_map     pinned: hand-typed table of result dtypes for every
                              (tokens, probs) dtype pair, values equal to the
                              plain permutation cast to those dtypes.
fused-op output conventions   PARITY UNPINNED: what the closed vendor kernels
  (second output of           ``aclnnMoeTokenPermute`` / ``aclnnGroupedMatmul``
  npu_moe_token_permute,      really return for dropped rows, rows past the
  rows past last offset)      last group offset and their bf16 rounding order
                              cannot be observed from the reference tree; the
                              conventions used here are stated where defined.
"""
from __future__ import annotations

import torch

__all__ = [
    "permute", "row_id_map", "fused_permute", "unpermute", "fused_unpermute",
    "permute_backward", "unpermute_backward", "grouped_matmul", "gmm_split",
    "gmm", "gmm_backward", "groupmatmul_add_fp32", "swiglu", "swiglu_backward",
    "sort_chunks_by_idxs", "experts_computation", "moe_layer", "route_topk",
    "permute_routing_map", "fused_permute_routing_map", "unpermute_routing_map",
]


# --------------------------------------------------------------------------
# permute
# --------------------------------------------------------------------------
def permute(tokens, indices, num_out_tokens=None):
    """Index-mode permute of the torch path.

    Follows mindspeed/core/transformer/moe/moe_utils.py:199-210 and its twin
    mindspeed/fsdp/distributed/expert_parallel/utils.py:10-15: flatten the
    ``[T, k]`` expert ids token-major, stable-sort them (the reference sorts
    the float cast; ids are small integers so the cast is exact), optionally
    keep the first ``num_out_tokens`` entries, and gather ``tokens`` rows by
    ``sorted_indices // k``.

    Returns ``(permuted_tokens, sorted_indices)`` with ``sorted_indices`` in
    the forward convention: ``sorted_indices[r]`` is the flat ``t*k+j``
    position that produced output row ``r``.
    """
    topk = 1 if indices.dim() == 1 else indices.size(1)
    flat = indices.reshape(-1)
    sorted_indices = torch.sort(flat.float(), stable=True)[1]
    if num_out_tokens is not None:
        sorted_indices = sorted_indices[:num_out_tokens]
    permuted = tokens.index_select(0, sorted_indices // topk)
    return permuted, sorted_indices


def row_id_map(indices):
    """Inverse of the full forward order: ``map[t*k+j]`` = output row.

    This is the convention of the fused op's second output (int32, always
    ``T*k`` long, never sliced): mindspeed/ops/csrc/cann/
    npu_moe_token_permute.cpp:81-85 allocates it that way and
    npu_moe_token_unpermute.cpp:109-113 recovers ``T`` as ``len/topk``.
    """
    flat = indices.reshape(-1)
    fwd = torch.sort(flat.float(), stable=True)[1]
    inv = torch.empty_like(fwd)
    inv[fwd] = torch.arange(fwd.numel(), dtype=fwd.dtype)
    return inv.to(torch.int32)


def fused_permute(tokens, indices, num_out_tokens=None):
    """What ``npu_moe_token_permute`` returns, stated with the torch path.

    Shapes and the ``num_out_tokens`` rule follow mindspeed/ops/csrc/cann/
    npu_moe_token_permute.cpp:78-86: ``n > 0 -> min(n, T*k)``, otherwise
    ``n + T*k``; ``permuted`` has that many rows, the map keeps ``T*k``
    entries and flat positions whose row is ``>=`` that count are dropped.
    """
    flat_size = indices.numel()
    n = 0 if num_out_tokens is None else int(num_out_tokens)
    actual = min(n, flat_size) if n > 0 else n + flat_size
    permuted, _ = permute(tokens, indices, actual)
    return permuted, row_id_map(indices)


# --------------------------------------------------------------------------
# unpermute
# --------------------------------------------------------------------------
def unpermute(permuted_tokens, sorted_indices, probs=None):
    """Forward-order unpermute of the torch path.

    Follows mindspeed/core/transformer/moe/moe_utils.py:213-241 (twin:
    mindspeed/fsdp/distributed/expert_parallel/utils.py:26-34): scatter the
    rows back with ``index_copy_`` into a zero buffer, view as ``[T, k, H]``,
    multiply by ``probs[..., None]`` in the input dtype and sum over ``k``.
    """
    if probs is not None:
        num_unpermuted = probs.numel()
        topk = probs.size(1)
    else:
        num_unpermuted = permuted_tokens.size(0)
        topk = 1
    buf = torch.zeros([num_unpermuted, permuted_tokens.shape[-1]],
                      dtype=permuted_tokens.dtype)
    buf.index_copy_(0, sorted_indices.long(), permuted_tokens)
    buf = buf.reshape(-1, topk, permuted_tokens.size(-1))
    if probs is not None:
        buf = buf * probs.unsqueeze(-1)
    return buf.sum(dim=1)


def fused_unpermute(permuted_tokens, row_map, probs=None):
    """``npu_moe_token_unpermute`` stated with the torch path.

    ``row_map`` is the inverse map (see :func:`row_id_map`); entries that
    point past ``permuted_tokens`` are dropped rows and contribute zero.
    ``out[t] = sum_j probs[t, j] * permuted[row_map[t*k+j]]`` — the gather
    form of moe_utils.py:230-239.  Output shape ``[len(row_map)/k, H]`` as in
    mindspeed/ops/csrc/cann/npu_moe_token_unpermute.cpp:108-114.
    """
    topk = 1 if probs is None else probs.size(1)
    rm = row_map.long()
    rows = permuted_tokens.size(0)
    keep = rm < rows
    gathered = permuted_tokens.index_select(0, rm.clamp(max=max(rows - 1, 0))) \
        if rows > 0 else permuted_tokens.new_zeros(rm.numel(), permuted_tokens.size(-1))
    gathered = gathered * keep.unsqueeze(-1).to(gathered.dtype)
    buf = gathered.reshape(-1, topk, permuted_tokens.size(-1))
    if probs is not None:
        buf = buf * probs.unsqueeze(-1)
    return buf.sum(dim=1)


def permute_backward(grad_permuted, row_map, topk):
    """``grad_tokens[t] = sum_j grad_permuted[row_map[t*k+j]]``.

    The autograd of the ``index_select`` in moe_utils.py:209; shapes as in
    mindspeed/ops/csrc/cann/npu_moe_token_permute.cpp:113-115.
    """
    rm = row_map.long()
    rows = grad_permuted.size(0)
    keep = (rm < rows).unsqueeze(-1).to(grad_permuted.dtype)
    g = grad_permuted.index_select(0, rm.clamp(max=max(rows - 1, 0))) * keep
    return g.reshape(-1, topk, grad_permuted.size(-1)).sum(dim=1)


def unpermute_backward(grad_out, permuted_tokens, row_map, probs=None):
    """Gradients of :func:`fused_unpermute`.

    ``grad_permuted[row_map[t*k+j]] = probs[t,j] * grad_out[t]`` and
    ``grad_probs[t,j] = <grad_out[t], permuted[row_map[t*k+j]]>``; output
    shapes follow mindspeed/ops/csrc/cann/npu_moe_token_unpermute.cpp:140-141.
    The dot product is taken in fp32 and rounded to the probs dtype.
    """
    topk = 1 if probs is None else probs.size(1)
    rm = row_map.long()
    rows, hidden = permuted_tokens.shape
    keep = rm < rows
    g = grad_out.repeat_interleave(topk, dim=0)
    if probs is not None:
        g = g * probs.reshape(-1, 1)
    grad_permuted = torch.zeros_like(permuted_tokens)
    grad_permuted.index_copy_(0, rm[keep], g[keep])
    grad_probs = None
    if probs is not None:
        gathered = permuted_tokens.index_select(0, rm.clamp(max=max(rows - 1, 0))).float()
        gathered = gathered * keep.unsqueeze(-1)
        dots = (gathered.reshape(-1, topk, hidden) * grad_out.float().unsqueeze(1)).sum(-1)
        grad_probs = dots.to(probs.dtype)
    return grad_permuted, grad_probs


# --------------------------------------------------------------------------
# grouped matmul
# --------------------------------------------------------------------------
def grouped_matmul(inputs, m_split, weights):
    """Per-group ``torch.matmul`` loop.

    Follows mindspeed/ops/grouped_matmul.py:85-133: accepts ``[E, K, N]`` or
    ``[E, N, K]`` weights (the latter is transposed), zero-initialises the
    output, takes group boundaries from ``cumsum(m_split)``.
    """
    batch, input_dim = inputs.shape
    if weights.shape[1] == input_dim:
        out_dim = weights.shape[2]
    else:
        out_dim = weights.shape[1]
        weights = weights.transpose(1, 2)
    out = torch.zeros((batch, out_dim), dtype=inputs.dtype)
    bounds = [0] + torch.cumsum(torch.as_tensor(m_split), dim=0).tolist()
    for i in range(len(bounds) - 1):
        s, e = bounds[i], bounds[i + 1]
        out[s:e, :] = torch.matmul(inputs[s:e, :], weights[i])
    return out


def gmm_split(x, weight, group_sizes, group_type):
    """The reference unit test's own oracle for ``npu_gmm``.

    Follows tests_extend/unit_tests/ops/cann/test_npu_gmm.py:36-49: for
    ``group_type == 0`` split ``x`` by rows; for ``group_type == 2`` split
    ``x`` on its last dim and ``weight`` on dim 0; multiply per expert and
    concatenate on dim 0.
    """
    group_sizes = [int(v) for v in group_sizes]
    if group_type == 0:
        xs = list(x.split(group_sizes, dim=0))
        ws = [weight[i] for i in range(len(group_sizes))]
    elif group_type == 2:
        xs = list(x.split(group_sizes, dim=-1))
        ws = list(weight.split(group_sizes, dim=0))
    else:
        raise ValueError("group_type must be 0 or 2")
    outs = [xs[i] @ ws[i] for i in range(len(group_sizes))]
    return torch.cat(outs, dim=0)


def _counts(group_list, group_list_type):
    gl = [int(v) for v in (group_list.tolist() if torch.is_tensor(group_list) else group_list)]
    if group_list_type == 0:
        return [gl[0]] + [gl[i] - gl[i - 1] for i in range(1, len(gl))] if gl else []
    return gl


def gmm(x, weight, group_list, group_type=0, group_list_type=0):
    """``npu_gmm`` (cumulative ``group_list``) / ``npu_gmm_v2`` (counts).

    Output shapes follow mindspeed/ops/csrc/cann/gmm.cpp:48-54: ``[M, N]`` for
    ``group_type`` 0 and ``[E, K, N]`` for ``group_type`` 2.  Rows past the
    last offset are zero (the torch path zero-initialises its output,
    mindspeed/ops/grouped_matmul.py:115); an empty group gives a zero
    ``[K, N]`` block (tests_extend/unit_tests/ops/cann/test_npu_gmm.py:105-113).
    """
    counts = _counts(group_list, group_list_type)
    if group_type == 0:
        out = torch.zeros((x.size(0), weight.size(-1)), dtype=x.dtype)
        used = sum(counts)
        if used:
            out[:used] = gmm_split(x[:used], weight, counts, 0)
        return out
    used = sum(counts)
    res = gmm_split(x[:, :used], weight[:used], counts, 2)
    return res.reshape(len(counts), x.size(0), weight.size(-1))


def gmm_backward(grad, x, weight, group_list, group_list_type=0):
    """``dx = gmm(grad, w^T, 0)``, ``dw = gmm(x^T, grad, 2).reshape(w.shape)``.

    Follows mindspeed/ops/csrc/cann/gmm.cpp:169-200.
    """
    dx = gmm(grad, weight.transpose(-1, -2), group_list, 0, group_list_type)
    dw = gmm(x.transpose(-1, -2), grad, group_list, 2, group_list_type)
    return dx, dw.reshape(weight.shape)


def groupmatmul_add_fp32(x, dy, group_list, grad):
    """In place ``grad.view(E, K, N)[g] += x_g^T @ dy_g`` in fp32.

    Follows mindspeed/ops/npu_groupmatmul_add.py:11-16 and
    mindspeed/ops/csrc/atb/groupmatmul_add.cpp:39-64 (``transposeA=true``);
    ``group_list`` is cumulative.  The identity the reference test checks is
    ``out + dw`` (tests_extend/unit_tests/ops/atb/test_groupmatmul_add.py:24-33).
    """
    counts = _counts(group_list, 0)
    e = len(counts)
    view = grad.view(e, x.size(-1), dy.size(-1))
    s = 0
    for g, c in enumerate(counts):
        if c:
            view[g] += x[s:s + c].float().t() @ dy[s:s + c].float()
        s += c
    return grad


# --------------------------------------------------------------------------
# SwiGLU and chunk sort
# --------------------------------------------------------------------------
def swiglu(x, probs=None):
    """``silu(x[..., :F]) * x[..., F:]``, optionally times ``probs[:, None]``.

    The first half is the gate: mindspeed/core/transformer/moe/moe_feature/
    overlap/token_dispatcher.py:700-704 and mindspeed/fsdp/distributed/
    expert_parallel/dispatcher.py:94-95.  The probs product and the cast back
    follow mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:41-44.
    """
    gate, up = x.chunk(2, dim=-1)
    y = torch.nn.functional.silu(gate) * up
    if probs is not None:
        y = (y * probs.reshape(-1, 1)).to(x.dtype)
    return y


def swiglu_backward(grad_y, x, probs=None):
    """Gradient of :func:`swiglu` w.r.t. ``x`` (and ``probs``), fp32 math."""
    gate, up = x.float().chunk(2, dim=-1)
    g = grad_y.float()
    sig = torch.sigmoid(gate)
    act = gate * sig
    grad_probs = None
    if probs is not None:
        grad_probs = (g * act * up).sum(-1).to(probs.dtype)
        g = g * probs.float().reshape(-1, 1)
    dgate = g * up * (sig * (1 + gate * (1 - sig)))
    dup = g * act
    return torch.cat([dgate, dup], dim=-1).to(x.dtype), grad_probs


def sort_chunks_by_idxs(inp, split_sizes, sorted_idxs, probs=None):
    """Reorder contiguous row chunks.

    Follows mindspeed/core/transformer/moe/moe_feature/overlap/
    moe_common.py:377-398: ``cat([split(inp, split_sizes)[i] for i in
    sorted_idxs])`` and the same for ``probs``.
    """
    sizes = [int(v) for v in (split_sizes.tolist() if torch.is_tensor(split_sizes) else split_sizes)]
    order = [int(v) for v in (sorted_idxs.tolist() if torch.is_tensor(sorted_idxs) else sorted_idxs)]
    chunks = torch.split(inp, sizes, dim=0)
    out = torch.cat([chunks[i] for i in order], dim=0)
    out_probs = None
    if probs is not None:
        pch = torch.split(probs, sizes, dim=0)
        out_probs = torch.cat([pch[i] for i in order], dim=0)
    return out, out_probs


# --------------------------------------------------------------------------
# whole single-rank pipeline
# --------------------------------------------------------------------------
def experts_computation(hidden, split_list, gate_up_weights, down_weights,
                        act_fn=torch.nn.functional.silu):
    """Follows mindspeed/fsdp/distributed/expert_parallel/dispatcher.py:93-97."""
    gate, up = grouped_matmul(hidden, split_list, gate_up_weights).chunk(2, dim=-1)
    act = act_fn(gate) * up
    return grouped_matmul(act, split_list, down_weights)


def moe_layer(hidden, top_k_index, top_k_weights, gate_up_weights, down_weights):
    """``dispatch_mlp_combine`` with one rank (no all-to-all).

    Follows mindspeed/fsdp/distributed/expert_parallel/dispatcher.py:37-52,
    81-113 with ``ep_size == 1``: permute by expert, grouped MLP, weighted
    unpermute.  With one rank the second permute/unpermute pair is the
    identity (rows are already expert-major).
    """
    num_experts = gate_up_weights.size(0)
    tokens_per_expert = torch.bincount(top_k_index.reshape(-1), minlength=num_experts)
    permuted, sorted_indices = permute(hidden, top_k_index)
    out = experts_computation(permuted, tokens_per_expert, gate_up_weights, down_weights)
    return unpermute(out, sorted_indices, top_k_weights)


def route_topk(logits, topk):
    """softmax -> top-k -> renormalise (input generation only).

    Follows mindspeed/core/transformer/moe/moe_utils.py:429-435.
    """
    probs_full = torch.softmax(logits.float(), dim=-1)
    p, idx = torch.topk(probs_full, topk, dim=-1)
    p = p / p.sum(dim=-1, keepdim=True)
    return p, idx


# --------------------------------------------------------------------------
# routing-map (mask) mode
# --------------------------------------------------------------------------
def permute_routing_map(tokens, routing_map, probs=None, num_out_tokens=None, drop_and_pad=False):
    """Megatron-LM core_r0.12 ``moe_utils.permute`` (the function the reference's
    mindspeed/core/fusions/fused_moe_permute.py:65-66 falls back to and that the vendor op behind
    mindspeed/te/pytorch/permutation.py:23-24 replaces).

    ``routing_map`` ``[T, E]`` bool, ``probs`` ``[T, E]``.  Returns
    ``(permuted_tokens, permuted_probs, sorted_indices)`` with ``sorted_indices`` the token id of every
    output row, rows expert-major and token-ascending.  ``drop_and_pad``: ``capacity = num_out_tokens // E``
    rows per expert, chosen by a stable descending argsort of the transposed map (routed tokens first,
    non-routed tokens as padding)."""
    num_tokens, _ = tokens.shape
    num_experts = routing_map.shape[1]
    permuted_probs = None
    if drop_and_pad and num_out_tokens is not None:
        capacity = num_out_tokens // num_experts
        rm = routing_map.to(torch.int8).T.contiguous()
        sorted_indices = rm.argsort(dim=-1, descending=True, stable=True)[:, :capacity].contiguous().view(-1)
        if probs is not None:
            probs_t = probs.T.contiguous().view(-1)
            dim0 = torch.arange(num_experts).unsqueeze(-1)
            flat = (dim0 * num_tokens + sorted_indices.view(num_experts, capacity)).view(-1)
            permuted_probs = probs_t.index_select(0, flat)
    else:
        rm = routing_map.bool().T.contiguous()
        token_indices = torch.arange(num_tokens).unsqueeze(0).expand(num_experts, -1)
        sorted_indices = token_indices.masked_select(rm)
        if probs is not None:
            # same expression as mindspeed/core/transformer/moe/moe_feature/overlap/token_dispatcher.py:451-453
            permuted_probs = probs.T.contiguous().masked_select(rm)
    permuted = tokens.index_select(0, sorted_indices)
    return permuted, permuted_probs, sorted_indices


def fused_permute_routing_map(tokens, routing_map, probs=None, num_out_tokens=None, drop_and_pad=False):
    """The reference's ``permute`` hook with ``fused=True``
    (mindspeed/core/fusions/fused_moe_permute.py:17-47,58-63): when exactly one of ``tokens`` / ``probs`` is
    fp32, both are promoted to fp32, permuted, and *both* results are cast to the dtype of the operand that was
    not fp32 (``convert_tensors_to_fp32_if_needed`` / ``restore_original_dtype``).  Any other dtype pair, and a
    call without ``probs``, goes through unchanged."""
    original = None
    if isinstance(tokens, torch.Tensor) and isinstance(probs, torch.Tensor) and \
            ((tokens.dtype == torch.float32) ^ (probs.dtype == torch.float32)):
        original = probs.dtype if tokens.dtype == torch.float32 else tokens.dtype
        tokens, probs = tokens.to(torch.float32), probs.to(torch.float32)
    permuted, permuted_probs, sorted_indices = permute_routing_map(tokens, routing_map, probs, num_out_tokens,
                                                                   drop_and_pad)
    if original is not None:
        permuted = permuted.to(original)
        permuted_probs = permuted_probs.to(original) if permuted_probs is not None else None
    return permuted, permuted_probs, sorted_indices


def unpermute_routing_map(permuted_tokens, sorted_indices, restore_shape, probs=None, routing_map=None,
                          drop_and_pad=False):
    """Megatron-LM core_r0.12 ``moe_utils.unpermute``; its non-padded branch is restated in-tree at
    mindspeed/core/transformer/moe/unpermute_without_activation.py:44-62: rows are scaled by their
    permuted probability and scatter-added into ``zeros(restore_shape)`` by token id; the product and
    the sum are in the promoted dtype, the result is cast back to the input dtype."""
    _, hidden = restore_shape
    input_dtype = permuted_tokens.dtype
    if probs is not None:
        if drop_and_pad:
            num_experts = routing_map.size(1)
            capacity = sorted_indices.size(0) // num_experts
            num_unpermuted = probs.size(0)
            probs_t = probs.T.contiguous().view(-1)
            dim0 = torch.arange(num_experts).unsqueeze(-1)
            flat = (dim0 * num_unpermuted + sorted_indices.view(num_experts, capacity)).view(-1)
            permuted_probs = probs_t.index_select(0, flat)
        else:
            permuted_probs = probs.T.contiguous().masked_select(routing_map.T.contiguous())
        permuted_tokens = permuted_tokens * permuted_probs.unsqueeze(-1)
    out = torch.zeros(restore_shape, dtype=permuted_tokens.dtype)
    out = out.scatter_add(0, sorted_indices.unsqueeze(1).expand(-1, hidden), permuted_tokens)
    return out.to(input_dtype)
