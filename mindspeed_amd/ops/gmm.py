"""``npu_gmm`` / ``npu_gmm_v2`` on MI355X.

Mirrors mindspeed/ops/gmm.py: the same parameter verification
(``npu_gmm_param_verification``, gmm.py:103-136), the same dispatcher schemas
(mindspeed/op_builder/gmm_builder.py:90-93,131-133), the same autograd split
into forward / dX / dW (gmm.py:20-99, mindspeed/ops/csrc/cann/gmm.cpp:169-293)
and the same raw list-in / list-out module that
``GMMFunction.builder.load()`` returns (gmm.cpp:295-309).  Every product is one
call of the ``ms_gmm`` C-ABI entry point on strided views; nothing is
transposed in memory.
"""
from __future__ import annotations

import ctypes
import os

import torch

from .. import _lib, flop_counter
from ._kernels import K, _plain
from .npu_groupmatmul_add import npu_groupmatmul_add_fp32

__all__ = ["npu_gmm", "npu_gmm_v2", "GMMFunction"]


# --------------------------------------------------------------------------
# raw kernel call
# --------------------------------------------------------------------------
def _unit_stride_view(t: torch.Tensor) -> torch.Tensor:
    """Return ``t`` if one of its two matrix strides is 1, else a contiguous copy."""
    if t.stride(-1) == 1 or t.stride(-2) == 1 or t.size(-1) <= 1 or t.size(-2) <= 1:
        return t
    return t.contiguous()


def _group_list_tensor(group_list, device) -> torch.Tensor:
    if isinstance(group_list, torch.Tensor):
        if group_list.device != device:
            group_list = group_list.to(device)
        return group_list.contiguous()
    return torch.tensor(list(group_list), dtype=torch.int64, device=device)


def gmm_raw(x, weight, group_list, group_type, group_list_type, out=None, accumulate=False):
    """One grouped matmul on the current stream.

    group_type 0: ``x [M, K]``, ``weight [E, K, N]`` -> ``[M, N]``.
    group_type 2: ``x [K, M]``, ``weight [M, N]`` -> ``[E, K, N]``.
    ``out``: optional preallocated contiguous result (fp32, or x's dtype); fp32 with ``accumulate`` adds the
    result in place.
    """
    _lib.require_device(x, "x")
    _lib.require_device(weight, "weight")
    dev = x.device
    _lib.dtype_code(x.dtype, "x")
    if weight.dtype != x.dtype:
        raise TypeError(f"x and weight must have the same dtype, got {x.dtype} and {weight.dtype}")
    gl = _group_list_tensor(group_list, dev)
    if gl.dtype != torch.int64 or gl.dim() != 1:
        raise TypeError("group_list must be a one-dimensional int64 tensor")
    num_groups = gl.numel()
    x = _unit_stride_view(x)
    weight = _unit_stride_view(weight)
    if group_type == 0:
        if x.dim() != 2 or weight.dim() != 3:
            raise ValueError(f"group_type 0 needs x [M, K] and weight [E, K, N], got {tuple(x.shape)}, {tuple(weight.shape)}")
        m, k = x.shape
        if weight.size(0) != num_groups or weight.size(1) != k:
            raise ValueError(f"weight {tuple(weight.shape)} does not match x {tuple(x.shape)} and {num_groups} groups")
        n = weight.size(2)
        w_strides = (weight.stride(0), weight.stride(1), weight.stride(2))
        out_shape = (m, n)
    elif group_type == 2:
        if x.dim() != 2 or weight.dim() != 2:
            raise ValueError(f"group_type 2 needs x [K, M] and weight [M, N], got {tuple(x.shape)}, {tuple(weight.shape)}")
        k, m = x.shape
        if weight.size(0) != m:
            raise ValueError(f"weight {tuple(weight.shape)} does not match x {tuple(x.shape)}")
        n = weight.size(1)
        w_strides = (0, weight.stride(0), weight.stride(1))
        out_shape = (num_groups, k, n)
    else:
        raise ValueError(f"group_type must be 0 or 2, got {group_type}")
    if out is None:
        return K.gmm(x, weight, gl, group_type, group_list_type)
    numel = out_shape[0] * out_shape[1] * (out_shape[2] if len(out_shape) == 3 else 1)
    if out.dtype not in (torch.float32, x.dtype) or not out.is_contiguous() or out.numel() != numel:
        raise ValueError("out must be a contiguous tensor of the result's size, fp32 or of x's dtype")
    if accumulate and out.dtype != torch.float32:
        raise ValueError("accumulate needs an fp32 out")
    K.gmm_out(x, weight, gl, group_type, group_list_type, out, bool(accumulate))
    return out


def gmm_raw_weight_list(x, weights, group_list, group_list_type, transposed=False):
    """``y[rows of group g] = x[rows of g] @ W_g`` with one separately allocated matrix per group.

    ``weights``: sequence of 2-D tensors of one shape, dtype and stride pattern; ``W_g = weights[g]``
    (``[K, N]``), or ``weights[g].T`` with ``transposed`` (``[N, K]`` parameters read in place).
    """
    _lib.require_device(x, "x")
    weights = list(weights)
    if not weights:
        raise RuntimeError("Neither x nor weight could be empty")
    dev = x.device
    _lib.dtype_code(x.dtype, "x")
    x = _unit_stride_view(x)
    first = weights[0]
    views = []
    for i, w in enumerate(weights):
        _lib.require_device(w, f"weight[{i}]")
        if w.dtype != x.dtype:
            raise TypeError(f"x and weight must have the same dtype, got {x.dtype} and {w.dtype}")
        if w.dim() != 2 or w.shape != first.shape:
            raise ValueError(f"every weight must be a matrix of shape {tuple(first.shape)}, weight[{i}] is {tuple(w.shape)}")
        v = w.t() if transposed else w
        if v.stride(0) != 1 and v.stride(1) != 1:
            v = (w.contiguous().t() if transposed else w.contiguous())
        views.append(v)
    strides = (views[0].stride(0), views[0].stride(1))
    for i, v in enumerate(views):
        if (v.stride(0), v.stride(1)) != strides:
            views[i] = v.contiguous() if strides[1] == 1 else v.t().contiguous().t()
    gl = _group_list_tensor(group_list, dev)
    if gl.dtype != torch.int64 or gl.dim() != 1:
        raise TypeError("group_list must be a one-dimensional int64 tensor")
    num_groups = gl.numel()
    if x.dim() != 2 or len(views) != num_groups or views[0].size(0) != x.size(1):
        raise ValueError(f"{len(views)} weights of shape {tuple(views[0].shape)} do not match x {tuple(x.shape)} "
                         f"and {num_groups} groups")
    return K.gmm_weight_list(x, views, gl, group_list_type)


# dX and dW of one grouped matmul are independent; each is a full-chip kernel whose last round of tiles may leave
# compute units idle.  With MINDSPEED_AMD_OVERLAP_WGRAD=1 the weight-gradient product is launched on a second stream
# (default priority) between two joins with the caller's stream, so its tiles fill the other kernel's tail and vice
# versa.  Off by default: since the dX launch cuts its last-round tail tiles into parts along the reduction it ends
# with a full round by itself, and running the two kernels one after the other measures 0.8 % faster per step on the
# Mixtral and DeepSeek-share shapes (equal on the Qwen-like one).
OVERLAP_WGRAD = os.environ.get("MINDSPEED_AMD_OVERLAP_WGRAD", "0") != "0"
_side_streams = {}


def _side_stream(device) -> torch.cuda.Stream:
    key = (device.type, device.index if device.index is not None else torch.cuda.current_device())
    s = _side_streams.get(key)
    if s is None:
        s = torch.cuda.Stream(device=device)
        _side_streams[key] = s
    return s


class _beside:
    """``with _beside(tensor) as side:`` runs the body on the side stream after everything queued so far on the
    current stream; ``side.join()`` (call it after queueing the main-stream work that should overlap)
    makes the current stream wait for the body.  Results of the body should live in memory that was
    allocated on the caller's stream beforehand.  Without overlap (disabled,
    or while ops are being event-timed one by one) the body simply runs on the current stream."""

    def __init__(self, like: torch.Tensor):
        device = like.device
        self.active = OVERLAP_WGRAD and not flop_counter.timing_active() and not _tracing(like)
        self.main = torch.cuda.current_stream(device) if self.active else None
        self.side = _side_stream(device) if self.active else None
        self.ctx = None

    def __enter__(self):
        if self.active:
            self.side.wait_stream(self.main)
            self.ctx = torch.cuda.stream(self.side)
            self.ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False

    def again(self):
        """A further ``with`` block on the side stream, ordered after what the caller's stream holds now (and,
        being the same stream, after the earlier block)."""
        return self

    def join(self):
        if self.active:
            self.main.wait_stream(self.side)


def _add_group_bias(y, bias, group_list, group_list_type):
    """``y[rows of group g] += bias[g]`` (forward only, as in the reference: mindspeed/ops/gmm.py:27-28 refuses a bias
    that requires a gradient).  ``bias [E, N]``, fp16 / bf16 / fp32.  Plain torch ops on the device, nothing read
    back: the sum is formed in fp32 from the product as the grouped matmul stored it and rounded once more, rows past
    the last offset stay zero.  How the vendor kernel rounds (it may add before its only rounding) is not stated in the
    reference tree."""
    _lib.require_device(bias, "bias")
    gl = _group_list_tensor(group_list, y.device)
    num_groups = gl.numel()
    if bias.dim() != 2 or bias.size(0) != num_groups or bias.size(1) != y.size(1):
        raise ValueError(f"bias must be [{num_groups}, {y.size(1)}], got {tuple(bias.shape)}")
    # the group ends exactly as the kernels derive them: a cumulative list never runs backwards and never past the
    # row count, negative counts read as zero (and the vector handed to searchsorted is then always sorted)
    m = y.size(0)
    if group_list_type == 0:
        ends = torch.cummax(gl, dim=0).values.clamp(0, m)
    else:
        ends = gl.clamp(0, m).cumsum(dim=0).clamp(max=m)
    rows = torch.arange(m, device=y.device)
    group = torch.searchsorted(ends, rows, right=True)
    covered = (group < num_groups).unsqueeze(1)
    picked = bias.index_select(0, group.clamp(max=num_groups - 1)).float()
    return torch.where(covered, y.float() + picked, y.float()).to(y.dtype)


class _RawGmmModule:
    """Stand-in for the pybind module of mindspeed/ops/csrc/cann/gmm.cpp:295-309.

    Callers such as mindspeed/core/transformer/moe/grouped_matmul_util.py:140-184
    use ``GMMFunction.builder.load().npu_gmm([x], [w], bias, group_list, group_type,
    group_list_type)`` and get lists back.
    """

    @staticmethod
    def npu_gmm(x, weight, bias, group_list, group_type, group_list_type):
        if len(x) != 1 or len(weight) != 1:
            raise RuntimeError("Neither x nor weight could be empty; single-tensor (split_item=3) form only.")
        group_type = group_type if group_type is not None else 0
        y = gmm_raw(x[0], weight[0], group_list, group_type, group_list_type or 0)
        if bias:
            if len(bias) != 1 or group_type != 0:
                raise ValueError("bias: one [E, N] tensor, with the split on rows (group_type 0) only")
            y = _add_group_bias(y, bias[0], group_list, group_list_type or 0)
        return [y]

    @staticmethod
    def npu_gmm_backward(grad, x, weight, group_list, group_list_type):
        # gmm.cpp:169-246: dx = gmm(grad, w^T, 0); dw = gmm(x^T, grad, 2).reshape(w.shape)
        glt = group_list_type or 0
        # The result is allocated on the caller's stream: a block that belonged to the side stream's pool
        # would have its release deferred until the caller's stream is done with it, and the next step's
        # request on the side stream would then go to the driver for fresh memory.
        w = weight[0]
        num_groups = len(group_list) if not isinstance(group_list, torch.Tensor) else group_list.numel()
        dw = torch.empty((num_groups, x[0].size(-1), grad[0].size(-1)), dtype=x[0].dtype, device=x[0].device)
        with _beside(grad[0]) as side:
            gmm_raw(x[0].transpose(-1, -2), grad[0], group_list, 2, glt, out=dw)
        dx = gmm_raw(grad[0], w.transpose(-1, -2), group_list, 0, glt)
        side.join()
        return [dx], [dw.reshape(w.shape)], []

    @staticmethod
    def npu_gmm_backward_fusion(grad, weight, group_list, group_list_type):
        # gmm.cpp:248-293: dx only.
        dx = gmm_raw(grad[0], weight[0].transpose(-1, -2), group_list, 0, group_list_type or 0)
        return [dx], [], []


class _Builder:
    _module = _RawGmmModule()

    def load(self):
        _lib.load()
        return self._module


def _tracing(t: torch.Tensor) -> bool:
    """True when ``t`` is a meta / fake tensor or a compiler is tracing: no kernel runs then, so there is nothing
    to overlap and no stream to fork."""
    return t.device.type == "meta" or torch.compiler.is_compiling() or \
        isinstance(t, torch._subclasses.fake_tensor.FakeTensor)


class GMMFunction(torch.autograd.Function):
    """Autograd node of ``npu_gmm`` / ``npu_gmm_v2`` (mindspeed/ops/gmm.py:20-99).

    ``apply(original_weight, x, weight, bias, group_args)`` with ``group_args = (group_list, group_type,
    gemm_fusion, group_list_type, group_list_data_type)``; gradients ``(None, dx, dw, dbias, None)``.  A list
    ``group_list`` (data type 0) rides on the context, a tensor one is saved with the other tensors.
    """
    builder = _Builder()
    builder2 = _Builder()

    @staticmethod
    def _module(group_list_type):
        return (GMMFunction.builder if group_list_type == 0 else GMMFunction.builder2).load()

    @staticmethod
    def forward(ctx, original_weight, x, weight, bias, group_args):
        group_list, group_type, gemm_fusion, group_list_type, group_list_data_type = group_args
        if bias is not None and bias.requires_grad:
            raise ValueError("Bias is not supported to compute gradient!")
        if (x.requires_grad or weight.requires_grad) and group_type != 0:
            raise ValueError("group_type must be zero to compute gradients of x and weight!")
        (y,) = GMMFunction._module(group_list_type).npu_gmm(
            [x], [weight], [] if bias is None else [bias], group_list, group_type, group_list_type)
        list_form = group_list_data_type == 0
        ctx.save_for_backward(x, weight, original_weight, *(() if list_form else (group_list,)))
        ctx.group_list = group_list if list_form else None
        ctx.gemm_fusion = gemm_fusion
        ctx.group_list_type = group_list_type
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, weight, original_weight, *rest = ctx.saved_tensors
        group_list = rest[0] if rest else ctx.group_list
        module = GMMFunction._module(ctx.group_list_type)
        if not ctx.gemm_fusion:
            (dx,), (dw,), dbias = module.npu_gmm_backward([grad_y], [x], [weight], group_list, ctx.group_list_type)
            return None, dx, dw, (dbias[0] if dbias else None), None
        # gemm_fusion (gmm.py:56-89): the weight gradient is added into original_weight.main_grad (fp32) by the
        # accumulate form of the dW product, here on the side stream beside dX; what autograd gets for the weight is
        # a placeholder (zeros if the parameter asks for it) and the flag the optimizer wrapper looks at is set.
        with _beside(grad_y) as side:
            offsets = group_list if ctx.group_list_type == 0 else torch.cumsum(group_list, dim=0)
            npu_groupmatmul_add_fp32(x, grad_y, offsets, original_weight.main_grad)
        (dx,), _, dbias = module.npu_gmm_backward_fusion([grad_y], [weight], group_list, ctx.group_list_type)
        side.join()
        placeholder = None
        if hasattr(original_weight, "grad_added_to_main_grad"):
            make = torch.zeros if getattr(weight, "zero_out_wgrad", False) else torch.empty
            placeholder = make(weight.shape, dtype=x.dtype, device=x.device, requires_grad=False)
            original_weight.grad_added_to_main_grad = True
        return None, dx, placeholder, (dbias[0] if dbias else None), None


def npu_gmm_param_verification(x, weight, *, bias=None, group_list=None, group_type=0, group_list_type=0):
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"arg0 must be a torch.Tensor, got {type(x)}.")
    if not isinstance(weight, torch.Tensor):
        raise TypeError(f"arg1 must be a torch.Tensor, got {type(weight)}.")
    if not isinstance(bias, (torch.Tensor, type(None))):
        raise TypeError(f"bias must be a torch.Tensor or None, got {type(bias)}.")
    if group_list_type == 0:
        if not (
            isinstance(group_list, (torch.Tensor, type(None)))
            or (isinstance(group_list, list) and all(isinstance(v, int) for v in group_list))
        ):
            raise TypeError(f"group_list must be a List of int64, torch.Tensor or None, got {type(group_list)}.")
    else:
        if not isinstance(group_list, (torch.Tensor, type(None))):
            raise TypeError(f"group_list must be a torch.Tensor or None, got {type(group_list)}.")
    if isinstance(group_list, torch.Tensor):
        if len(group_list.shape) > 1:
            raise ValueError(f"If group_list is not None, it must be an one-dimensional tensor, "
                             f"got dimension of group_list: {len(group_list.shape)}!")
        if group_list.dtype != torch.int64:
            raise TypeError(f"group_list must be a List of int64, got group_list type: {type(group_list)}, "
                            f"dtype: {group_list.dtype}!")
    if not isinstance(group_type, (int, type(None))):
        raise TypeError(f"group_type must be an int or None, got {type(group_type)}.")
    x_device = x.device
    device_warning = "Expected all tensors to be on the same device, but found at least two devices"
    if weight.device != x_device:
        raise RuntimeError(f"{device_warning}, {x_device}(arg0) and {weight.device}(arg1)!")
    if bias is not None and bias.device != x_device:
        raise RuntimeError(f"{device_warning}, {x_device}(arg0) and {bias.device}(bias)!")
    if isinstance(group_list, torch.Tensor) and group_list.device != x_device:
        raise RuntimeError(f"{device_warning}, {x_device}(arg0) and {group_list.device}(group_list)!")


# --------------------------------------------------------------------------
# dispatcher registration: same schemas as the reference, namespace "mindspeed"
# --------------------------------------------------------------------------
def _define_library():
    try:
        lib = torch.library.Library("mindspeed", "DEF")
    except RuntimeError:
        # another provider (the reference itself) already owns the namespace
        lib = torch.library.Library("mindspeed", "FRAGMENT")
    defined = []
    for schema in (
        "npu_gmm.List(Tensor? original_weight, Tensor x, Tensor weight, *, Tensor? bias=None, "
        "int[]? group_list=None, int? group_type=0, bool? gemm_fusion=False) -> Tensor",
        "npu_gmm.Tensor(Tensor? original_weight, Tensor x, Tensor weight, *, Tensor? bias=None, "
        "Tensor? group_list=None, int? group_type=0, bool? gemm_fusion=False) -> Tensor",
        "npu_gmm_v2.Tensor(Tensor? original_weight, Tensor x, Tensor weight, *, Tensor? bias=None, "
        "Tensor? group_list=None, int? group_type=0, bool? gemm_fusion=False) -> Tensor",
    ):
        try:
            lib.define(schema)
            defined.append(schema.split("(")[0])
        except RuntimeError:
            pass
    return lib, defined


_LIBRARY, _DEFINED = _define_library()


def _npu_gmm(original_weight, x, weight, *, bias=None, group_list=None, group_type=0, gemm_fusion=False):
    group_list_data_type = 1 if isinstance(group_list, (torch.Tensor, type(None))) else 0
    group_args = (group_list, group_type, gemm_fusion, 0, group_list_data_type)
    return GMMFunction.apply(original_weight, x, weight, bias, group_args)


def _npu_gmm_v2(original_weight, x, weight, *, bias=None, group_list=None, group_type=0, gemm_fusion=False):
    group_args = (group_list, group_type, gemm_fusion, 1, 1)
    return GMMFunction.apply(original_weight, x, weight, bias, group_args)


for _name, _fn in (("npu_gmm.List", _npu_gmm), ("npu_gmm.Tensor", _npu_gmm), ("npu_gmm_v2.Tensor", _npu_gmm_v2)):
    if _name in _DEFINED:
        # The implementation is an autograd.Function over dispatcher ops that carry their own device and fake
        # (meta) kernels (ops/_kernels.py), so it is registered as a composite: autograd sees through it, and on
        # meta / fake tensors it decomposes into those ops and yields the output shape the reference's explicit
        # Meta registrations compute (mindspeed/op_builder/gmm_builder.py:101-106,141-146).  torch refuses a
        # direct Meta kernel next to a composite one.
        _LIBRARY.impl(_name, _fn, "CompositeImplicitAutograd")


def _npu_gmm_common(original_weight, x, weight, *, bias=None, group_list=None, group_type=0, group_list_type=0,
                    gemm_fusion=False):
    support_dtype = [torch.float16, torch.bfloat16, torch.float32]
    if isinstance(weight, torch.Tensor) and weight.dtype not in support_dtype:
        raise TypeError(f"Only support non quant case, but got weight dtype {weight.dtype}.")
    npu_gmm_param_verification(x, weight, bias=bias, group_list=group_list, group_type=group_type,
                               group_list_type=group_list_type)
    if group_list is None:
        raise ValueError("group_list is required: the single-tensor (split_item=3) form needs group boundaries")
    if bias is not None and group_type != 0:
        raise ValueError("bias is supported with the split on rows (group_type 0) only")
    # Plain device tensors in eager mode: the composite op's implementation directly (what the dispatcher would
    # decompose to), without the boxing of a Python-registered op; anything that may want to see the call goes
    # through the dispatcher.
    direct = _plain((original_weight, x, weight, bias, group_list if isinstance(group_list, torch.Tensor) else None))
    if group_list_type == 0:
        fn = _npu_gmm if direct else torch.ops.mindspeed.npu_gmm
    elif group_list_type == 1:
        fn = _npu_gmm_v2 if direct else torch.ops.mindspeed.npu_gmm_v2
    else:
        raise ValueError(f"group_list_type must be 0 or 1, but got {group_list_type}.")
    return fn(original_weight, x, weight, bias=bias, group_list=group_list, group_type=group_type,
              gemm_fusion=gemm_fusion)


def npu_gmm(x, weight, *, bias=None, group_list=None, group_type=0, gemm_fusion=False, original_weight=None):
    """Grouped matmul; ``group_list`` holds cumulative row offsets (list or int64 tensor)."""
    return _npu_gmm_common(original_weight, x, weight, bias=bias, group_list=group_list, group_type=group_type,
                           group_list_type=0, gemm_fusion=gemm_fusion)


def npu_gmm_v2(x, weight, *, bias=None, group_list=None, group_type=0, gemm_fusion=False, original_weight=None):
    """Grouped matmul; ``group_list`` holds per-group row counts (int64 tensor)."""
    return _npu_gmm_common(original_weight, x, weight, bias=bias, group_list=group_list, group_type=group_type,
                           group_list_type=1, gemm_fusion=gemm_fusion)
