"""``Ops.gmm``: the object Megatron's ``grouped_gemm_util.ops`` is replaced by.

Mirrors mindspeed/core/fusions/grouped_matmul.py:5-21,35-50 (registered over
``megatron.core.transformer.moe.grouped_gemm_util.ops`` by
mindspeed/features_manager/fusions/grouped_matmul.py:8-16).  Megatron's expert modules call
``gg.ops.gmm(x, w, tokens_per_expert, trans_b=False)`` (and MindSpeed's own with ``gemm_fusion`` /
``original_weight``, mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:113-120,146-153) with
``batch_sizes`` = rows per expert.
"""
from __future__ import annotations

import torch

__all__ = ["Ops", "grouped_gemm_is_available", "assert_grouped_gemm_is_available", "get_device_capability"]


class Ops:
    @staticmethod
    def gmm(a, b, batch_sizes, trans_b=False, gemm_fusion=False, original_weight=None):
        """``y[rows of expert g] = a[rows of g] @ b[g]`` (``b[g].T`` with ``trans_b``).

        ``batch_sizes``: rows per expert, an int64 tensor on the device or on the host (Megatron keeps it on
        either).  It is summed where it lives and, if that is the host, sent over without waiting: the kernels take
        cumulative offsets from device memory and nothing is read back.  ``trans_b`` passes the weight as a strided
        view; no transposed copy is made.
        """
        from ..ops.gmm import npu_gmm

        if trans_b:
            # the reference writes b.t(), which torch defines for matrices only; a stack of matrices is
            # transposed per expert
            b = b.t() if b.dim() <= 2 else b.transpose(-1, -2)
        group_list = torch.cumsum(batch_sizes, dim=0).to(a.device, non_blocking=True)
        return npu_gmm(a, b, bias=None, group_list=group_list, group_type=0, gemm_fusion=gemm_fusion,
                       original_weight=original_weight)


def grouped_gemm_is_available():
    """True when the grouped matmul op can be imported and its kernel library is built."""
    try:
        from ..ops.gmm import npu_gmm  # noqa: F401
        from .. import _lib
        _lib.load()
        return True
    except (ImportError, RuntimeError, OSError):
        return False


def assert_grouped_gemm_is_available():
    if not grouped_gemm_is_available():
        raise ImportError("from mindspeed_amd.ops.gmm import npu_gmm failed, or libmindspeed_amd.so is not built.")


def get_device_capability(device=None):
    """Megatron gates its grouped-GEMM path on compute capability >= (8, 0); the reference answers (9, 0)
    (mindspeed/core/fusions/grouped_matmul.py:49-50) and so does this."""
    return 9, 0
