"""``npu_groupmatmul_add_fp32`` on MI355X.

Mirrors mindspeed/ops/npu_groupmatmul_add.py:11-16 (kernel call:
mindspeed/ops/csrc/atb/groupmatmul_add.cpp:39-64, ``transposeA=true``): in
place ``grad.view(E, K, N)[g] += x_g^T @ dy_g`` with fp32 accumulation, the
dW kernel's accumulate epilogue.
"""
from __future__ import annotations

import torch

__all__ = ["npu_groupmatmul_add_fp32"]


def npu_groupmatmul_add_fp32(x, dy, grouplist, grad):
    from .gmm import gmm_raw  # deferred: gmm.py imports this module

    if grad.dtype != torch.float32:
        raise TypeError(f"grad must be float32, got {grad.dtype}")
    if not grad.is_contiguous():
        raise ValueError("grad must be contiguous (it is updated in place)")
    if not isinstance(grouplist, torch.Tensor):
        grouplist = torch.tensor(list(grouplist), dtype=torch.int64, device=x.device)
    num_groups = grouplist.shape[0]
    if grad.numel() != num_groups * x.shape[-1] * dy.shape[-1]:
        raise ValueError(f"grad has {grad.numel()} elements, expected {num_groups}x{x.shape[-1]}x{dy.shape[-1]}")
    gmm_raw(x.transpose(-1, -2), dy, grouplist, 2, 0, out=grad, accumulate=True)
    return None
