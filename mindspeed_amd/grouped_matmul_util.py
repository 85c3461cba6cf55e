"""``BaseGMMFunction`` / ``BF16GMMFunction``: the grouped matmul as an autograd node with separable products.

Mirrors mindspeed/core/transformer/moe/grouped_matmul_util.py:41-184.  The class exposes the three products of a
grouped matmul as class methods over the raw module that ``GMMFunction.builder.load()`` returns —

* ``op_forward(ctx, x, weight, group_list, group_list_type, bias)``  ``x @ w[g]``            (:140-148)
* ``op_dx(ctx, grad, weight, group_list, group_list_type)``          ``grad @ w[g]^T``        (:150-168)
* ``op_dw(ctx, x, grad, group_list, group_list_type)``               ``x_g^T @ grad_g``       (:170-184)
* ``op_gmm_add(x, weight, grad, group_list, weight_param)``          ``main_grad += x^T grad`` (:110-135)

— so that a schedule can run the weight gradient later than dX.  ``WeightGradStore`` is the queue the reference's
forward/backward-overlap schedules use for that (mindspeed/core/transformer/moe/moe_feature/fb_overlap/modules/
weight_grad_store.py:29-58,86-108): with ``WeightGradStore.is_decoupleBlock`` the backward pass returns dX at once,
parks ``(x, grad, group_list)`` in the queue, and ``WeightGradStore.pop()`` later runs the K-grouped matmul by
itself and adds the result to ``weight_param.main_grad`` (directly into the fp32 buffer with
``gemm_gradient_accumulation_fusion``).  The fp8 / mxfp8 subclasses of the reference are outside this path.
"""
from __future__ import annotations

import torch

from .ops.gmm import GMMFunction
from .ops.npu_groupmatmul_add import npu_groupmatmul_add_fp32

__all__ = ["BaseGMMFunction", "BF16GMMFunction", "WeightGradStore", "get_gmm_op_cls", "get_gmm_quant_func", "gmm_settings"]


class _Settings:
    """The two command-line switches the reference reads from its global arguments (``get_args()``)."""
    gemm_gradient_accumulation_fusion = False
    overlap_grad_reduce = False


gmm_settings = _Settings()


def get_gmm_quant_func():
    """No quantised grouped matmul on this path (grouped_matmul_util.py:19-31 returns None without fp8 too)."""
    return None


def get_gmm_op_cls():
    return BF16GMMFunction


class WeightGradStore:
    """Queue of deferred weight-gradient products (weight_grad_store.py:29-58,86-108, expert weights only)."""
    cache = []
    is_decoupleBlock = False

    @classmethod
    def put(cls, total_input, grad_output, weight, sequence_parallel=False, in_row=False):
        cls.cache.append((total_input, grad_output, weight, sequence_parallel, in_row))

    @classmethod
    def pop(cls, all_entries=True):
        """Run the parked products in order, on the current stream.  ``all_entries=False``: only the oldest."""
        while cls.cache:
            cls.overlap_matmul(cls.cache.pop(0))
            if not all_entries:
                break

    @classmethod
    def overlap_matmul(cls, entry):
        total_input, grad_output, weight, _sequence_parallel, _in_row = entry
        ctx, inputs, group_list, group_list_type, weight_shape = total_input
        gmm_cls = get_gmm_op_cls()
        if gmm_settings.gemm_gradient_accumulation_fusion and not getattr(weight, "is_hot_experts", False):
            gmm_cls.gmm_add_impl(inputs, grad_output, group_list, weight, weight_shape)
        else:
            (grad_weight,) = GMMFunction.builder.load().npu_gmm([inputs.t()], [grad_output], [], group_list, 2, 0)
            if getattr(weight, "is_hot_experts", False):
                weight.grad = grad_weight.view(-1, weight.shape[-1])
            else:
                weight.main_grad.data.add_(grad_weight.view(weight.main_grad.shape))

    @classmethod
    def clear(cls):
        cls.cache = []
        cls.is_decoupleBlock = False


class BaseGMMFunction(torch.autograd.Function):
    @classmethod
    def gmm_apply(cls, x, weight, bias, tokens_per_expert, weight_param):
        if isinstance(tokens_per_expert, list):
            tokens_per_expert = torch.tensor(tokens_per_expert, device=x.device, dtype=torch.int64)
        group_list = torch.cumsum(tokens_per_expert, dim=0)
        return cls.apply(x, weight, bias, group_list, weight_param)

    @classmethod
    def forward(cls, ctx, x, weight, bias, group_list, weight_param, group_list_type=0):
        if isinstance(group_list, torch.Tensor):
            if group_list.device != x.device:
                group_list = group_list.to(x.device)
        else:
            group_list = torch.tensor(group_list, device=x.device, dtype=torch.int64)
        output = cls.op_forward(ctx, x, weight, group_list, group_list_type, bias=bias)
        ctx.save_for_backward(x, weight, group_list)
        ctx.weight_param = weight_param
        ctx.group_list_type = group_list_type
        return output[0]

    @classmethod
    def backward(cls, ctx, grad_outputs):
        x, weight, group_list = ctx.saved_tensors
        weight_param = ctx.weight_param
        group_list_type = ctx.group_list_type
        grad_outputs = grad_outputs.contiguous()
        dx = cls.op_dx(ctx, grad_outputs, weight, group_list, group_list_type)[0]
        if WeightGradStore.is_decoupleBlock:
            # dW is not computed here: its operands wait in the queue for WeightGradStore.pop()
            WeightGradStore.put([ctx, x, group_list, group_list_type, weight.shape], grad_outputs, weight_param,
                                sequence_parallel=False, in_row=False)
            if hasattr(weight_param, "grad_added_to_main_grad") and gmm_settings.overlap_grad_reduce:
                weight_param.skip_grad_accum = True
            grad_weights = None
        elif gmm_settings.gemm_gradient_accumulation_fusion:
            grad_weights = cls.op_gmm_add(x, weight, grad_outputs, group_list, weight_param)
        else:
            grad_weights = cls.op_dw(ctx, x, grad_outputs, group_list, group_list_type)[0]
        return dx, grad_weights, None, None, None, None

    @classmethod
    def op_forward(cls, ctx, x, weight, group_list, group_list_type=0, bias=None):
        raise NotImplementedError

    @classmethod
    def op_dx(cls, ctx, grad, weight, group_list, group_list_type=0, bias=None):
        raise NotImplementedError

    @classmethod
    def op_dw(cls, ctx, x, grad, group_list, group_list_type=0, bias=None):
        raise NotImplementedError

    @classmethod
    def op_gmm_add(cls, x, weight, grad, group_list, weight_param):
        cls.gmm_add_impl(x, grad, group_list, weight_param, weight.shape)
        if not hasattr(weight_param, "grad_added_to_main_grad"):
            return None
        make = torch.zeros if getattr(weight, "zero_out_wgrad", False) else torch.empty
        grad_weights = make(weight.shape, dtype=x.dtype, device=x.device, requires_grad=False)
        weight_param.grad_added_to_main_grad = True
        return grad_weights

    @classmethod
    def gmm_add_impl(cls, x, grad, group_list, weight_param, weight_shape):
        npu_groupmatmul_add_fp32(x, grad, group_list, weight_param.main_grad)


class BF16GMMFunction(BaseGMMFunction):
    """The three products through the raw module's list-in / list-out ``npu_gmm`` (cumulative ``group_list``)."""

    @classmethod
    def op_forward(cls, ctx, x, weight, group_list, group_list_type=0, bias=None):
        return GMMFunction.builder.load().npu_gmm([x], [weight], bias or [], group_list, 0, group_list_type)

    @classmethod
    def op_dx(cls, ctx, grad, weight, group_list, group_list_type=0, bias=None):
        # rearrange(weight, 'n h f -> n f h'): a strided view, read in place by the kernel
        weight = weight.transpose(1, 2) if weight.dim() == 3 else weight.t()
        return GMMFunction.builder.load().npu_gmm([grad], [weight], bias or [], group_list, 0, group_list_type)

    @classmethod
    def op_dw(cls, ctx, x, grad, group_list, group_list_type=0, bias=None):
        return GMMFunction.builder.load().npu_gmm([x.t()], [grad], bias or [], group_list, 2, group_list_type)
