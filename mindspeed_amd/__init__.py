"""mindspeed_amd — MI355X-native MoE expert hot path behind the ``mindspeed.ops`` API.

The public surface mirrors the reference module paths:

* ``mindspeed_amd.ops.npu_moe_token_permute.npu_moe_token_permute``
* ``mindspeed_amd.ops.npu_moe_token_unpermute.npu_moe_token_unpermute``
* ``mindspeed_amd.ops.gmm.npu_gmm`` / ``npu_gmm_v2``
* ``mindspeed_amd.ops.npu_groupmatmul_add.npu_groupmatmul_add_fp32``

All of them call hand-written HIP kernels through the C ABI of
``libmindspeed_amd.so``; nothing here computes on the CPU.
"""
__version__ = "0.1.0"
