"""``MindSpeedTEGroupedLinear`` on MI355X: the per-expert-parameter module API.

Mirrors mindspeed/te/pytorch/module/grouped_linear.py:47-98 (``MindSpeedTEGroupedLinearGMM``) and the
module of :131-249 as far as the expert path goes: ``num_gemms`` separate parameters ``weight{i}`` of
shape ``[output_size, input_size]``, ``forward(x, m_splits) -> (output, None)`` with ``m_splits`` the
per-expert row counts.  The reference makes a transposed contiguous copy of every weight on every forward
(:235) and hands the list to ``torch_npu.npu_grouped_matmul``; here the parameters are read in place
through ``ms_gmm_weight_list`` (one device pointer per expert) and the weight gradients come out of one
``[E, out, in]`` buffer as views, in the parameters' own orientation.  Tensor-parallel partitioning,
checkpoint sharding and the MXFP8 recipes of the reference module are outside this path.
"""
from __future__ import annotations

from typing import Sequence

import torch
from torch.nn.parameter import Parameter

from .gmm import gmm_raw, gmm_raw_weight_list

__all__ = ["MindSpeedTEGroupedLinearGMM", "MindSpeedTEGroupedLinear"]


class MindSpeedTEGroupedLinearGMM(torch.autograd.Function):
    """``apply(input, m_split, group_list_type, *weights)`` with ``weights[i]`` of shape ``[N, K]``.

    (The reference's signature also carries the list of transposed copies it has just made,
    grouped_linear.py:47-50,236-238; no copies are made here, so the parameters are the only weights.)
    """

    @staticmethod
    def forward(ctx, input_tensor: torch.Tensor, m_split, group_list_type, *weights) -> torch.Tensor:
        if not isinstance(m_split, torch.Tensor):   # grouped_linear.py:53-56
            m_split = torch.tensor(list(m_split), device=input_tensor.device, dtype=torch.int64)
        ctx.group_list = m_split
        ctx.group_list_type = group_list_type
        ctx.save_for_backward(input_tensor, *weights)
        return gmm_raw_weight_list(input_tensor, weights, m_split, group_list_type, transposed=True)

    @staticmethod
    def backward(ctx, grad_output):
        inp = ctx.saved_tensors[0]
        weights = ctx.saved_tensors[1:]
        grad_output = grad_output.contiguous()
        # grouped_linear.py:78-86: dX = dY @ W_g, W_g = weight{g} [N, K] as stored
        grad = gmm_raw_weight_list(grad_output, weights, ctx.group_list, ctx.group_list_type, transposed=False)
        # grouped_linear.py:87-96 (reduction split): dW_g = dY_g^T @ x_g, [N, K] like the parameter
        grad_weight = gmm_raw(grad_output.t(), inp, ctx.group_list, 2, ctx.group_list_type)
        return (grad, None, None, *grad_weight.unbind(0))


class MindSpeedTEGroupedLinear(torch.nn.Module):
    """``num_gemms`` expert weights ``weight{i}`` ``[output_size, input_size]``; ``forward(x, m_splits)``
    returns ``(output, None)`` as the reference module does (grouped_linear.py:196-249)."""

    def __init__(self, num_gemms: int, input_size: int, output_size: int, *, init_method=None,
                 params_dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        self.num_gemms = num_gemms
        self.input_size = input_size
        self.output_size = output_size
        self.use_bias = False
        self.total_weight = []
        for i in range(num_gemms):
            w = Parameter(torch.empty(output_size, input_size, device=device, dtype=params_dtype))
            if init_method is not None:
                init_method(w)
            else:
                torch.nn.init.normal_(w, std=0.02)
            self.register_parameter(f"weight{i}", w)
            self.total_weight.append(w)

    def forward(self, x: torch.Tensor, m_splits: Sequence[int]):
        group_list_type = 1   # grouped_linear.py:234: counts
        output = MindSpeedTEGroupedLinearGMM.apply(x, m_splits, group_list_type, *self.total_weight)
        return output, None
