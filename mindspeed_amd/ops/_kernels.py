"""The C-ABI kernel calls as dispatcher ops (namespace ``mindspeed_amd``).

Every op here is one call of an entry point of ``libmindspeed_amd.so`` on tensors that the Python surface has
already validated.  Registering them with the dispatcher, each with a device kernel and a fake (meta) kernel
that only computes output shapes, is what lets the Python surface above them (autograd Functions, the
``mindspeed::npu_gmm`` ops) run on meta / fake tensors, i.e. be traced by ``torch.compile`` and shape-propagated
without touching the GPU — the job the reference's ``Meta`` registrations do for its ops
(mindspeed/op_builder/gmm_builder.py:101-106,141-146).

There is no CPU kernel: on CPU tensors the ops raise.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib, flop_counter

_LIB = torch.library.Library("mindspeed_amd", "DEF")


_DEVICE_FNS = {}


def _define(schema, device_fn, fake_fn):
    name = schema.split("(")[0]
    _DEVICE_FNS[name] = device_fn
    _LIB.define(schema)
    _LIB.impl(name, device_fn, "CUDA")
    torch.library.register_fake(f"mindspeed_amd::{name}", fake_fn, lib=_LIB)

    def _no_cpu(*args, **kwargs):
        raise RuntimeError(f"mindspeed_amd::{name} runs hand-written HIP kernels and needs tensors on an MI355X "
                           "(torch device type 'cuda' on ROCm); there is no CPU fallback.")
    _LIB.impl(name, _no_cpu, "CPU")


# ---- grouped matmul ----------------------------------------------------------------------------------------
def _gmm_dims(x, weight, group_list, group_type):
    """(m, k, n, weight strides (group, red, col), output shape) of one grouped matmul."""
    num_groups = group_list.numel()
    if group_type == 0:
        m, k = x.shape
        n = weight.size(2)
        return m, k, n, (weight.stride(0), weight.stride(1), weight.stride(2)), (m, n)
    k, m = x.shape
    n = weight.size(1)
    return m, k, n, (0, weight.stride(0), weight.stride(1)), (num_groups, k, n)


_GMM_WS = {}     # workspace bytes by problem: the size query is pure host arithmetic on these values


def _gmm_launch(x, weight, group_list, group_type, group_list_type, out, accumulate):
    lib = _lib.load()
    dev = x.device
    dtype = _lib.dtype_code(x.dtype, "x")
    m, k, n, w_strides, _ = _gmm_dims(x, weight, group_list, group_type)
    num_groups = group_list.numel()
    out_dtype = _lib.MS_FP32 if out.dtype == torch.float32 else dtype
    key = (num_groups, m, k, n, group_type, dtype, out_dtype, bool(accumulate))
    need = _GMM_WS.get(key)
    if need is None:
        nbytes = ctypes.c_size_t(0)
        _lib.check(lib.ms_gmm_workspace_size_split(num_groups, m, k, n, group_type, dtype, out_dtype,
                                                   1 if accumulate else 0, ctypes.byref(nbytes)),
                   "ms_gmm_workspace_size_split")
        if len(_GMM_WS) > 4096:
            _GMM_WS.clear()
        need = _GMM_WS[key] = nbytes.value
    ws = _lib.workspace(need, dev)
    # kernel flavour by operand layout: NN (forward), NT (weight read transposed: dX), TN (dW)
    if group_type == 2:
        kind = "gmm_dw"
    elif w_strides[1] == 1 and w_strides[2] != 1:
        kind = "gmm_dx"
    else:
        kind = "gmm_fwd"
    with _lib.on(dev), flop_counter.op(kind, flop_counter.gmm_flops(m, k, n), "flop", dev):
        _lib.check(lib.ms_gmm(
            _lib.stream_ptr(dev), _lib.ptr(x), x.stride(0), x.stride(1), _lib.ptr(weight), *w_strides,
            _lib.ptr(out), n, _lib.ptr(group_list), group_list_type, group_type, num_groups, m, k, n, dtype, out_dtype,
            1 if accumulate else 0, _lib.ptr(ws), ws.numel()), "ms_gmm")


def _gmm(x, weight, group_list, group_type, group_list_type):
    out = torch.empty(_gmm_dims(x, weight, group_list, group_type)[4], dtype=x.dtype, device=x.device)
    _gmm_launch(x, weight, group_list, group_type, group_list_type, out, False)
    return out


def _gmm_fake(x, weight, group_list, group_type, group_list_type):
    return x.new_empty(_gmm_dims(x, weight, group_list, group_type)[4])


def _gmm_out(x, weight, group_list, group_type, group_list_type, out, accumulate):
    _gmm_launch(x, weight, group_list, group_type, group_list_type, out, accumulate)


_define("gmm(Tensor x, Tensor weight, Tensor group_list, int group_type, int group_list_type) -> Tensor",
        _gmm, _gmm_fake)
_define("gmm_out(Tensor x, Tensor weight, Tensor group_list, int group_type, int group_list_type, "
        "Tensor(a!) out, bool accumulate) -> ()", _gmm_out, lambda *a: None)


# ---- token permute / unpermute -----------------------------------------------------------------------------
def _permute_shapes(tokens, indices, num_out, num_experts, want_sorted, want_counts):
    num_tokens, hidden = tokens.shape
    topk = 1 if indices.dim() == 1 else indices.size(1)
    return ((num_out, hidden), num_tokens * topk, num_out if want_sorted else 0,
            num_experts if (want_counts and num_experts > 0) else 0, topk)


def _permute(tokens, indices, num_out, num_experts, want_sorted, want_counts):
    lib = _lib.load()
    dev = tokens.device
    pshape, flat, nsorted, ncounts, topk = _permute_shapes(tokens, indices, num_out, num_experts, want_sorted,
                                                           want_counts)
    num_tokens, hidden = tokens.shape
    row_id_map = torch.empty(flat, dtype=torch.int32, device=dev)
    permuted = torch.empty(pshape, dtype=tokens.dtype, device=dev)
    sorted_idx = torch.empty(nsorted, dtype=torch.int32, device=dev)
    counts = torch.empty(ncounts, dtype=torch.int64, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_moe_token_permute_workspace_size(num_tokens, topk, num_experts, ctypes.byref(nbytes)),
               "ms_moe_token_permute_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    work = flop_counter.permute_bytes(num_tokens, topk, hidden, tokens.element_size(), indices.element_size(), num_out)
    with _lib.on(dev), flop_counter.op("permute", work, "byte", dev):
        _lib.check(lib.ms_moe_token_permute(
            _lib.stream_ptr(dev), _lib.ptr(tokens), _lib.ptr(indices), _lib.index_code(indices.dtype, "indices"),
            num_tokens, topk, hidden, _lib.dtype_code(tokens.dtype, "tokens"), num_out, num_experts,
            _lib.ptr(permuted), _lib.ptr(row_id_map), _lib.ptr(sorted_idx) if want_sorted else None,
            _lib.ptr(counts) if ncounts else None, _lib.ptr(ws), ws.numel()), "ms_moe_token_permute")
    return permuted, row_id_map, sorted_idx, counts


def _permute_fake(tokens, indices, num_out, num_experts, want_sorted, want_counts):
    pshape, flat, nsorted, ncounts, _ = _permute_shapes(tokens, indices, num_out, num_experts, want_sorted, want_counts)
    return (tokens.new_empty(pshape), tokens.new_empty(flat, dtype=torch.int32),
            tokens.new_empty(nsorted, dtype=torch.int32), tokens.new_empty(ncounts, dtype=torch.int64))


_define("moe_token_permute(Tensor tokens, Tensor indices, int num_out, int num_experts, bool want_sorted, "
        "bool want_counts) -> (Tensor, Tensor, Tensor, Tensor)", _permute, _permute_fake)


def _permute_grad(grad_permuted, row_id_map, num_tokens, topk):
    lib = _lib.load()
    dev = grad_permuted.device
    hidden = grad_permuted.size(1)
    grad_tokens = torch.empty((num_tokens, hidden), dtype=grad_permuted.dtype, device=dev)
    work = flop_counter.permute_grad_bytes(num_tokens, topk, hidden, grad_permuted.element_size(), grad_permuted.size(0))
    with _lib.on(dev), flop_counter.op("permute_grad", work, "byte", dev):
        _lib.check(lib.ms_moe_token_permute_grad(
            _lib.stream_ptr(dev), _lib.ptr(grad_permuted), _lib.ptr(row_id_map), num_tokens, topk, hidden,
            _lib.dtype_code(grad_permuted.dtype, "grad_permuted_tokens"), grad_permuted.size(0),
            _lib.ptr(grad_tokens)), "ms_moe_token_permute_grad")
    return grad_tokens


_define("moe_token_permute_grad(Tensor grad_permuted, Tensor row_id_map, int num_tokens, int topk) -> Tensor",
        _permute_grad, lambda g, r, num_tokens, topk: g.new_empty((num_tokens, g.size(1))))


def _kernel_probs(probs, token_dtype):
    """The kernels take probabilities in the tokens' dtype or in fp32; any other pair (fp16 beside bf16, 16-bit beside
    fp32 tokens) is widened to fp32 first, which is exact."""
    if probs is None or probs.dtype in (token_dtype, torch.float32):
        return probs
    return probs.float()


def _unpermute(permuted, row_id_map, probs, num_tokens, topk):
    lib = _lib.load()
    dev = permuted.device
    hidden = permuted.size(1)
    probs = _kernel_probs(probs, permuted.dtype)
    out = torch.empty((num_tokens, hidden), dtype=permuted.dtype, device=dev)
    work = flop_counter.unpermute_bytes(num_tokens, topk, hidden, permuted.element_size(), permuted.size(0))
    with _lib.on(dev), flop_counter.op("unpermute", work, "byte", dev):
        _lib.check(lib.ms_moe_token_unpermute(
            _lib.stream_ptr(dev), _lib.ptr(permuted), _lib.ptr(row_id_map), _lib.ptr(probs),
            _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0, num_tokens, topk, hidden,
            _lib.dtype_code(permuted.dtype, "permuted_tokens"), permuted.size(0), _lib.ptr(out)),
            "ms_moe_token_unpermute")
    return out


_define("moe_token_unpermute(Tensor permuted, Tensor row_id_map, Tensor? probs, int num_tokens, int topk) -> Tensor",
        _unpermute, lambda p, r, probs, num_tokens, topk: p.new_empty((num_tokens, p.size(1))))


def _unpermute_grad(permuted, grad_out, row_id_map, probs, num_tokens, topk, num_rows):
    """``permuted`` may be an empty tensor when there are no probabilities (it is only read for their gradient)."""
    lib = _lib.load()
    dev = grad_out.device
    hidden = grad_out.size(1)
    rows = num_rows
    probs_dtype = probs.dtype if probs is not None else None
    probs = _kernel_probs(probs, grad_out.dtype)
    grad_permuted = torch.empty((rows, hidden), dtype=grad_out.dtype, device=dev)
    grad_probs = torch.empty_like(probs) if probs is not None else torch.empty(0, dtype=grad_out.dtype, device=dev)
    mapped = min(rows, num_tokens * topk)
    if rows > mapped:
        grad_permuted.zero_()
    work = flop_counter.unpermute_grad_bytes(num_tokens, topk, hidden, grad_out.element_size(), rows, probs is not None)
    with _lib.on(dev), flop_counter.op("unpermute_grad", work, "byte", dev):
        _lib.check(lib.ms_moe_token_unpermute_grad(
            _lib.stream_ptr(dev), _lib.ptr(permuted) if probs is not None else None, _lib.ptr(grad_out),
            _lib.ptr(row_id_map), _lib.ptr(probs), _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0,
            num_tokens, topk, hidden,
            _lib.dtype_code(grad_out.dtype, "unpermuted_tokens_grad"), mapped, _lib.ptr(grad_permuted),
            _lib.ptr(grad_probs) if probs is not None else None), "ms_moe_token_unpermute_grad")
    if probs is not None and grad_probs.dtype != probs_dtype:
        grad_probs = grad_probs.to(probs_dtype)
    return grad_permuted, grad_probs


def _unpermute_grad_fake(permuted, grad_out, row_id_map, probs, num_tokens, topk, num_rows):
    return (grad_out.new_empty((num_rows, grad_out.size(1))),
            torch.empty_like(probs) if probs is not None else grad_out.new_empty(0))


_define("moe_token_unpermute_grad(Tensor permuted, Tensor grad_out, Tensor row_id_map, Tensor? probs, "
        "int num_tokens, int topk, int num_rows) -> (Tensor, Tensor)", _unpermute_grad, _unpermute_grad_fake)


# ---- SwiGLU --------------------------------------------------------------------------------------------------
def _swiglu(x2, probs):
    lib = _lib.load()
    rows, two_ffn = x2.shape
    ffn = two_ffn // 2
    y = torch.empty((rows, ffn), dtype=x2.dtype, device=x2.device)
    p_code = _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0
    with _lib.on(x2.device), flop_counter.op(
            "swiglu", flop_counter.swiglu_bytes(rows, ffn, x2.element_size()), "byte", x2.device):
        _lib.check(lib.ms_swiglu(_lib.stream_ptr(x2.device), _lib.ptr(x2), _lib.ptr(probs), p_code, rows, ffn,
                                 _lib.dtype_code(x2.dtype, "x"), _lib.ptr(y)), "ms_swiglu")
    return y


_define("swiglu(Tensor x, Tensor? probs) -> Tensor", _swiglu, lambda x2, probs: x2.new_empty((x2.size(0), x2.size(1) // 2)))


def _swiglu_grad(g, x2, probs):
    lib = _lib.load()
    rows, two_ffn = x2.shape
    ffn = two_ffn // 2
    gx = torch.empty_like(x2)
    gp = torch.empty_like(probs) if probs is not None else torch.empty(0, dtype=x2.dtype, device=x2.device)
    p_code = _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0
    with _lib.on(x2.device), flop_counter.op(
            "swiglu_grad", flop_counter.swiglu_bytes(rows, ffn, x2.element_size(), True), "byte", x2.device):
        _lib.check(lib.ms_swiglu_grad(_lib.stream_ptr(x2.device), _lib.ptr(g), _lib.ptr(x2), _lib.ptr(probs), p_code,
                                      rows, ffn, _lib.dtype_code(x2.dtype, "x"), _lib.ptr(gx),
                                      _lib.ptr(gp) if probs is not None else None), "ms_swiglu_grad")
    return gx, gp


_define("swiglu_grad(Tensor grad_y, Tensor x, Tensor? probs) -> (Tensor, Tensor)", _swiglu_grad,
        lambda g, x2, probs: (torch.empty_like(x2), torch.empty_like(probs) if probs is not None else x2.new_empty(0)))



# ---- routing-map (mask) form ---------------------------------------------------------------------------------
_ROUTING_MAP_WS = {}     # workspace bytes by (tokens, experts, mode): the size query is pure host arithmetic


def _routing_map_permute(tokens, routing_map, num_rows, drop_and_pad, want_counts):
    """``tokens`` may be None (maps only).  Returns (permuted or empty, row_id_map, sorted_flat, counts or empty)."""
    lib = _lib.load()
    dev = routing_map.device
    num_tokens, num_experts = routing_map.shape
    row_id_map = torch.empty(num_tokens * num_experts, dtype=torch.int32, device=dev)
    sorted_flat = torch.empty(num_rows, dtype=torch.int32, device=dev)
    counts = torch.empty(num_experts if want_counts else 0, dtype=torch.int64, device=dev)
    hidden, dtype_code, elem = 1, _lib.MS_FP32, 0
    if tokens is not None:
        hidden = tokens.size(1)
        dtype_code = _lib.dtype_code(tokens.dtype, "tokens")
        elem = tokens.element_size()
        permuted = torch.empty((num_rows, hidden), dtype=tokens.dtype, device=dev)
    else:
        permuted = torch.empty(0, dtype=torch.float32, device=dev)
    key = (num_tokens, num_experts, bool(drop_and_pad))
    need = _ROUTING_MAP_WS.get(key)
    if need is None:
        nbytes = ctypes.c_size_t(0)
        _lib.check(lib.ms_moe_routing_map_workspace_size(num_tokens, num_experts, int(drop_and_pad),
                                                         ctypes.byref(nbytes)), "ms_moe_routing_map_workspace_size")
        if len(_ROUTING_MAP_WS) > 4096:
            _ROUTING_MAP_WS.clear()
        need = _ROUTING_MAP_WS[key] = nbytes.value
    ws = _lib.workspace(need, dev)
    work = (num_tokens * hidden * elem + num_rows * hidden * elem if tokens is not None else 0) \
        + num_tokens * num_experts * (1 + 4) + num_rows * 4
    with _lib.on(dev), flop_counter.op("permute", work, "byte", dev):
        _lib.check(lib.ms_moe_routing_map_permute(
            _lib.stream_ptr(dev), _lib.ptr(tokens), _lib.ptr(routing_map), num_tokens, num_experts, hidden, dtype_code,
            num_rows, int(drop_and_pad), _lib.ptr(permuted) if tokens is not None else None, _lib.ptr(row_id_map),
            _lib.ptr(sorted_flat), _lib.ptr(counts) if want_counts else None, _lib.ptr(ws), ws.numel()),
            "ms_moe_routing_map_permute")
    return permuted, row_id_map, sorted_flat, counts


def _routing_map_permute_fake(tokens, routing_map, num_rows, drop_and_pad, want_counts):
    num_tokens, num_experts = routing_map.shape
    permuted = tokens.new_empty((num_rows, tokens.size(1))) if tokens is not None \
        else routing_map.new_empty(0, dtype=torch.float32)
    return (permuted, routing_map.new_empty(num_tokens * num_experts, dtype=torch.int32),
            routing_map.new_empty(num_rows, dtype=torch.int32),
            routing_map.new_empty(num_experts if want_counts else 0, dtype=torch.int64))


_define("routing_map_permute(Tensor? tokens, Tensor routing_map, int num_rows, bool drop_and_pad, bool want_counts) "
        "-> (Tensor, Tensor, Tensor, Tensor)", _routing_map_permute, _routing_map_permute_fake)


def _routing_map_probs(sorted_flat, probs, num_experts):
    """(permuted_probs or empty, sorted token ids int64)."""
    lib = _lib.load()
    dev = sorted_flat.device
    num_rows = sorted_flat.numel()
    permuted_probs = torch.empty(num_rows if probs is not None else 0,
                                 dtype=probs.dtype if probs is not None else torch.float32, device=dev)
    sorted_indices = torch.empty(num_rows, dtype=torch.int64, device=dev)
    with _lib.on(dev):
        _lib.check(lib.ms_moe_routing_map_probs(
            _lib.stream_ptr(dev), _lib.ptr(sorted_flat), num_rows, num_experts, _lib.ptr(probs),
            _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0,
            _lib.ptr(permuted_probs) if probs is not None else None, _lib.ptr(sorted_indices)),
            "ms_moe_routing_map_probs")
    return permuted_probs, sorted_indices


def _routing_map_probs_fake(sorted_flat, probs, num_experts):
    n = sorted_flat.numel()
    pp = probs.new_empty(n) if probs is not None else sorted_flat.new_empty(0, dtype=torch.float32)
    return pp, sorted_flat.new_empty(n, dtype=torch.int64)


_define("routing_map_probs(Tensor sorted_flat, Tensor? probs, int num_experts) -> (Tensor, Tensor)",
        _routing_map_probs, _routing_map_probs_fake)


def _routing_map_probs_grad(row_id_map, grad_permuted_probs, num_tokens, num_experts):
    lib = _lib.load()
    dev = row_id_map.device
    probs_grad = torch.empty((num_tokens, num_experts), dtype=grad_permuted_probs.dtype, device=dev)
    with _lib.on(dev):
        _lib.check(lib.ms_moe_routing_map_probs_grad(
            _lib.stream_ptr(dev), _lib.ptr(row_id_map), row_id_map.numel(), _lib.ptr(grad_permuted_probs),
            _lib.dtype_code(grad_permuted_probs.dtype, "probs"), grad_permuted_probs.numel(), _lib.ptr(probs_grad)),
            "ms_moe_routing_map_probs_grad")
    return probs_grad


_define("routing_map_probs_grad(Tensor row_id_map, Tensor grad_permuted_probs, int num_tokens, int num_experts) -> Tensor",
        _routing_map_probs_grad, lambda r, g, num_tokens, num_experts: g.new_empty((num_tokens, num_experts)))



# ---- grouped matmul with one weight matrix per group -----------------------------------------------------------
def _gmm_weight_list(x, weights, group_list, group_list_type):
    """``weights``: 2-D ``[K, N]`` views of one shape, dtype and stride pattern (the Python surface has made them so)."""
    lib = _lib.load()
    dev = x.device
    dtype = _lib.dtype_code(x.dtype, "x")
    num_groups = group_list.numel()
    m, k = x.shape
    n = weights[0].size(1)
    strides = (weights[0].stride(0), weights[0].stride(1))
    out = torch.empty((m, n), dtype=x.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_gmm_workspace_size(num_groups, m, 0, ctypes.byref(nbytes)), "ms_gmm_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    ptrs = (ctypes.c_void_p * num_groups)(*[v.data_ptr() for v in weights])
    kind = "gmm_dx" if strides[0] == 1 and strides[1] != 1 else "gmm_fwd"
    with _lib.on(dev), flop_counter.op(kind, flop_counter.gmm_flops(m, k, n), "flop", dev):
        _lib.check(lib.ms_gmm_weight_list(
            _lib.stream_ptr(dev), _lib.ptr(x), x.stride(0), x.stride(1), ptrs, strides[0], strides[1], _lib.ptr(out), n,
            _lib.ptr(group_list), group_list_type, num_groups, m, k, n, dtype, dtype, _lib.ptr(ws), ws.numel()),
            "ms_gmm_weight_list")
    return out


_define("gmm_weight_list(Tensor x, Tensor[] weights, Tensor group_list, int group_list_type) -> Tensor", _gmm_weight_list,
        lambda x, weights, group_list, group_list_type: x.new_empty((x.size(0), weights[0].size(1))))


# ---- grouped matmul with SwiGLU in its epilogue ------------------------------------------------------------------
def _gmm_swiglu(x, weight, group_list, group_list_type, probs, want_fc1):
    """``fc1 = grouped_matmul(x, weight)`` and ``act = silu(gate) * up * probs`` from one launch (contiguous 16-bit
    operands, checked by the Python surface).  Without ``want_fc1`` (nothing will be differentiated) the fc1 output is
    not stored at all and comes back empty."""
    lib = _lib.load()
    dev = x.device
    m, k = x.shape
    ffn = weight.size(2) // 2
    p_code = _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0
    fc1 = torch.empty((m, 2 * ffn) if want_fc1 else (0,), dtype=x.dtype, device=dev)
    act = torch.empty((m, ffn), dtype=x.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_gmm_workspace_size(group_list.numel(), m, 0, ctypes.byref(nbytes)), "ms_gmm_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    with _lib.on(dev), flop_counter.op("gmm_fwd_swiglu", flop_counter.gmm_flops(m, k, 2 * ffn), "flop", dev):
        _lib.check(lib.ms_gmm_swiglu(
            _lib.stream_ptr(dev), _lib.ptr(x), x.stride(0), x.stride(1), _lib.ptr(weight), weight.stride(0),
            weight.stride(1), weight.stride(2), _lib.ptr(fc1) if want_fc1 else None, 2 * ffn, _lib.ptr(act), ffn,
            _lib.ptr(probs), p_code,
            _lib.ptr(group_list), group_list_type, group_list.numel(), m, k, ffn, _lib.dtype_code(x.dtype, "x"),
            _lib.ptr(ws), ws.numel()), "ms_gmm_swiglu")
    return fc1, act


_define("gmm_swiglu(Tensor x, Tensor weight, Tensor group_list, int group_list_type, Tensor? probs, bool want_fc1) "
        "-> (Tensor, Tensor)",
        _gmm_swiglu, lambda x, weight, group_list, group_list_type, probs, want_fc1:
        (x.new_empty((x.size(0), weight.size(2)) if want_fc1 else (0,)), x.new_empty((x.size(0), weight.size(2) // 2))))


def _gmm_swiglu_grad(dy, w2, fc1, probs, group_list, group_list_type):
    """``d_fc1`` (and the probabilities' gradient) from ``dy``: the dX product of the second matmul with the SwiGLU
    backward on the saved ``fc1`` in its epilogue.  ``w2 [E, ffn, hidden]`` contiguous."""
    lib = _lib.load()
    dev = dy.device
    m, two_ffn = fc1.shape
    ffn = two_ffn // 2
    hidden = dy.size(1)
    num_groups = group_list.numel()
    d_fc1 = torch.empty_like(fc1)
    gp = torch.empty_like(probs) if probs is not None else torch.empty(0, dtype=fc1.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_gmm_swiglu_grad_workspace_size(num_groups, m, ffn, ctypes.byref(nbytes)),
               "ms_gmm_swiglu_grad_workspace_size")
    ws = _lib.workspace(nbytes.value, dev)
    wt = w2.transpose(1, 2)       # [E, hidden, ffn] view: element (k, n) of group g is w2[g, n, k]
    with _lib.on(dev), flop_counter.op("gmm_dx_swiglu", flop_counter.gmm_flops(m, hidden, ffn), "flop", dev):
        _lib.check(lib.ms_gmm_swiglu_grad(
            _lib.stream_ptr(dev), _lib.ptr(dy), dy.stride(0), dy.stride(1), _lib.ptr(w2), wt.stride(0),
            wt.stride(1), wt.stride(2), _lib.ptr(fc1), two_ffn, _lib.ptr(probs),
            _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0, _lib.ptr(d_fc1), two_ffn,
            _lib.ptr(gp) if probs is not None else None, _lib.ptr(group_list), group_list_type, num_groups, m, hidden,
            ffn, _lib.dtype_code(dy.dtype, "grad"), _lib.ptr(ws), ws.numel()), "ms_gmm_swiglu_grad")
    return d_fc1, gp


_define("gmm_swiglu_grad(Tensor dy, Tensor w2, Tensor fc1, Tensor? probs, Tensor group_list, int group_list_type) "
        "-> (Tensor, Tensor)", _gmm_swiglu_grad,
        lambda dy, w2, fc1, probs, group_list, group_list_type:
        (torch.empty_like(fc1), torch.empty_like(probs) if probs is not None else fc1.new_empty(0)))


# ---- chunk sort ------------------------------------------------------------------------------------------------------
def _sort_chunks(inp, split_sizes, sorted_idxs, probs, zero_fill):
    """Rows of ``inp`` (and entries of ``probs``) regrouped chunk by chunk, and the row map for the way back.
    ``zero_fill``: the outputs start as zeros (chunk lists that could not be checked on the host)."""
    lib = _lib.load()
    dev = inp.device
    rows, hidden = inp.shape
    new = torch.zeros_like if zero_fill else torch.empty_like
    out = new(inp)
    row_map = torch.empty(rows, dtype=torch.int32, device=dev)
    out_p = new(probs) if probs is not None else torch.empty(0, dtype=inp.dtype, device=dev)
    with _lib.on(dev):
        _lib.check(lib.ms_sort_chunks(
            _lib.stream_ptr(dev), _lib.ptr(inp), _lib.ptr(split_sizes), _lib.ptr(sorted_idxs),
            split_sizes.numel(), rows, hidden, _lib.dtype_code(inp.dtype, "input"), _lib.ptr(probs),
            _lib.dtype_code(probs.dtype, "probs") if probs is not None else 0, _lib.ptr(out),
            _lib.ptr(out_p) if probs is not None else None, _lib.ptr(row_map)), "ms_sort_chunks")
    return out, out_p, row_map


_define("sort_chunks(Tensor input, Tensor split_sizes, Tensor sorted_idxs, Tensor? probs, bool zero_fill) "
        "-> (Tensor, Tensor, Tensor)", _sort_chunks,
        lambda inp, split_sizes, sorted_idxs, probs, zero_fill:
        (torch.empty_like(inp), torch.empty_like(probs) if probs is not None else inp.new_empty(0),
         inp.new_empty((inp.size(0),), dtype=torch.int32)))


def _gather_rows(src, row_map, zero_fill):
    """``out[row_map[i]] = src[i]`` over the rows of a matrix or the entries of a vector (the chunk sort's way back)."""
    lib = _lib.load()
    dev = src.device
    out = torch.zeros_like(src) if zero_fill else torch.empty_like(src)
    rows = src.size(0)
    width = src.size(1) if src.dim() == 2 else 1
    with _lib.on(dev):
        _lib.check(lib.ms_gather_rows(_lib.stream_ptr(dev), _lib.ptr(src), _lib.ptr(row_map), rows, width,
                                      _lib.dtype_code(src.dtype, "grad"), 1, _lib.ptr(out)), "ms_gather_rows")
    return out


_define("gather_rows(Tensor src, Tensor row_map, bool zero_fill) -> Tensor", _gather_rows,
        lambda src, row_map, zero_fill: torch.empty_like(src))


def _chunk_sort_map(split_sizes, sorted_idxs, rows):
    """int32 ``[rows]``: entry ``r`` = output row of source row ``r`` under the chunk sort (-1 past the chunks)."""
    lib = _lib.load()
    dev = split_sizes.device
    row_id_map = torch.empty(rows, dtype=torch.int32, device=dev)
    with _lib.on(dev):
        _lib.check(lib.ms_chunk_sort_map(_lib.stream_ptr(dev), _lib.ptr(split_sizes), _lib.ptr(sorted_idxs),
                                         split_sizes.numel(), rows, _lib.ptr(row_id_map)), "ms_chunk_sort_map")
    return row_id_map


_define("chunk_sort_map(Tensor split_sizes, Tensor sorted_idxs, int rows) -> Tensor", _chunk_sort_map,
        lambda split_sizes, sorted_idxs, rows: split_sizes.new_empty((rows,), dtype=torch.int32))


def _move_rows(src, row_map, inverse, zero_fill):
    """``out[i] = src[row_map[i]]``, or with ``inverse`` ``out[row_map[i]] = src[i]``; rows or vector entries."""
    lib = _lib.load()
    dev = src.device
    out = torch.zeros_like(src) if zero_fill else torch.empty_like(src)
    rows = src.size(0)
    width = src.size(1) if src.dim() == 2 else 1
    with _lib.on(dev):
        _lib.check(lib.ms_gather_rows(_lib.stream_ptr(dev), _lib.ptr(src), _lib.ptr(row_map), rows, width,
                                      _lib.dtype_code(src.dtype, "input"), 1 if inverse else 0, _lib.ptr(out)),
                   "ms_gather_rows")
    return out


_define("move_rows(Tensor src, Tensor row_map, bool inverse, bool zero_fill) -> Tensor", _move_rows,
        lambda src, row_map, inverse, zero_fill: torch.empty_like(src))


def _zero_unmapped_rows(rows, sorted_flat):
    """Rows ``r`` of ``rows`` with ``sorted_flat[r] < 0`` become zeros, in place."""
    lib = _lib.load()
    dev = rows.device
    with _lib.on(dev):
        _lib.check(lib.ms_moe_zero_unmapped_rows(_lib.stream_ptr(dev), _lib.ptr(sorted_flat), rows.size(0), rows.size(1),
                                                 _lib.dtype_code(rows.dtype, "rows"), _lib.ptr(rows)),
                   "ms_moe_zero_unmapped_rows")


_define("zero_unmapped_rows(Tensor(a!) rows, Tensor sorted_flat) -> ()", _zero_unmapped_rows, lambda rows, sorted_flat: None)


# ---- how the Python surface reaches the ops -------------------------------------------------------------------------
# ``K.<op>(...)``.  On plain device tensors in eager mode that is the device kernel's Python function itself; whenever
# something may want to see the call — a compiler tracing, a dispatch or function mode on the stack (fake tensors,
# make_fx, profilers), a tensor subclass, a meta tensor — it goes through the dispatcher op of the same name, which
# routes to the same function for device tensors and to the fake kernel otherwise.  The direct call saves the boxing
# and schema matching of a Python-registered op (measured: about a third of the host time of a small layer step).
_len_dispatch_modes = torch._C._len_torch_dispatch_stack
_len_function_modes = torch._C._len_torch_function_stack


def _plain(args) -> bool:
    if _len_dispatch_modes() or _len_function_modes() or torch.compiler.is_compiling():
        return False
    for a in args:
        if a is None or a.__class__ is int or a.__class__ is bool:
            continue
        if a.__class__ is torch.Tensor:
            if a.device.type != "cuda":
                return False
        elif a.__class__ is torch.nn.Parameter:
            if a.device.type != "cuda":
                return False
        elif isinstance(a, (list, tuple)):
            if not _plain(a):
                return False
        elif isinstance(a, torch.Tensor):
            return False
    return True


class _Ops:
    def __init__(self):
        self._ns = torch.ops.mindspeed_amd

    def _bind(self, name, device_fn):
        op = getattr(self._ns, name)

        def call(*args):
            if _plain(args):
                return device_fn(*args)
            return op(*args)
        call.__name__ = name
        setattr(self, name, call)


K = _Ops()
for _name, _fn in _DEVICE_FNS.items():
    K._bind(_name, _fn)
