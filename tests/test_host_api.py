"""Host-side mirror of the reference interface: signatures, argument checks and
error types, and the rule that nothing computes off the GPU.  No GPU needed."""
import inspect
import os

import pytest
import torch

import mindspeed_amd.ops as ops
from mindspeed_amd.ops import gmm as gmm_mod


def test_signatures_match_reference():
    # mindspeed/ops/npu_moe_token_permute.py:13-18
    assert list(inspect.signature(ops.npu_moe_token_permute).parameters) == [
        "tokens", "indices", "num_out_tokens", "padded_mode"]
    # mindspeed/ops/npu_moe_token_unpermute.py:13-19
    assert list(inspect.signature(ops.npu_moe_token_unpermute).parameters) == [
        "permuted_tokens", "sorted_indices", "probs", "padded_mode", "restore_shape"]
    # mindspeed/ops/gmm.py:164,174
    for fn in (ops.npu_gmm, ops.npu_gmm_v2):
        sig = inspect.signature(fn)
        assert list(sig.parameters) == ["x", "weight", "bias", "group_list", "group_type", "gemm_fusion",
                                        "original_weight"]
        assert all(sig.parameters[p].kind is inspect.Parameter.KEYWORD_ONLY for p in list(sig.parameters)[2:])
    # mindspeed/ops/npu_groupmatmul_add.py:11
    assert list(inspect.signature(ops.npu_groupmatmul_add_fp32).parameters) == ["x", "dy", "grouplist", "grad"]


def test_dispatcher_schemas_registered():
    assert hasattr(torch.ops.mindspeed, "npu_gmm") and hasattr(torch.ops.mindspeed, "npu_gmm_v2")
    assert {"List", "Tensor"} <= set(torch.ops.mindspeed.npu_gmm.overloads())
    assert "Tensor" in torch.ops.mindspeed.npu_gmm_v2.overloads()


def test_no_cpu_fallback():
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    idx = torch.zeros(8, 2, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.npu_moe_token_permute(x, idx)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.npu_moe_token_unpermute(x, torch.zeros(8, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.npu_gmm(x, torch.randn(2, 16, 4, dtype=torch.bfloat16), group_list=[4, 8])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fused_swiglu(x)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.sort_chunks_by_idxs(x, [4, 4], [1, 0])


def test_sort_chunks_checks_host_lists():
    """Given on the host, the chunk sizes must sum to the row count and the order must be a permutation, as the
    reference's split / cat require (moe_common.py:377-398)."""
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="permutation"):
        ops.sort_chunks_by_idxs(x, [4, 4], [0, 0])
    with pytest.raises(RuntimeError, match="permutation"):
        ops.sort_chunks_by_idxs(x, torch.tensor([4, 4]), torch.tensor([1, 2]))
    with pytest.raises(RuntimeError, match="do not sum"):
        ops.sort_chunks_by_idxs(x, [4, 3], [1, 0])
    with pytest.raises(RuntimeError, match="do not sum"):
        ops.sort_chunks_by_idxs(x, [9, -1], [1, 0])


def test_permute_argument_checks():
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="padded_mode"):
        ops.npu_moe_token_permute(x, torch.zeros(8, 2, dtype=torch.int64), padded_mode=True)
    with pytest.raises(TypeError, match="int64 or int32"):
        ops.npu_moe_token_permute(x, torch.zeros(8, 2, dtype=torch.int16))
    with pytest.raises(TypeError, match="tokens"):
        ops.npu_moe_token_permute(x.to(torch.float64), torch.zeros(8, 2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="2 dimensional"):
        ops.npu_moe_token_permute(x.view(2, 4, 16), torch.zeros(8, 2, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="2 or 1 dimensional"):
        ops.npu_moe_token_permute(x, torch.zeros(8, 2, 1, dtype=torch.int64))


def test_unpermute_argument_checks():
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="padded_mode"):
        ops.npu_moe_token_unpermute(x, torch.zeros(8, dtype=torch.int32), padded_mode=True)
    with pytest.raises(TypeError, match="int32"):
        ops.npu_moe_token_unpermute(x, torch.zeros(8, dtype=torch.int64))
    with pytest.raises(RuntimeError, match="1 dimensional"):
        ops.npu_moe_token_unpermute(x, torch.zeros(4, 2, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="probs should be 2 dimensional"):
        ops.npu_moe_token_unpermute(x, torch.zeros(8, dtype=torch.int32), torch.ones(8, dtype=torch.bfloat16))


def test_gmm_argument_checks():
    # mindspeed/ops/gmm.py:103-150
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    w = torch.randn(2, 16, 4, dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="arg0"):
        ops.npu_gmm([1], w, group_list=[4, 8])
    with pytest.raises(TypeError, match="arg1"):
        ops.npu_gmm(x, None, group_list=[4, 8])
    with pytest.raises(TypeError, match="bias"):
        ops.npu_gmm(x, w, bias=3, group_list=[4, 8])
    with pytest.raises(TypeError, match="group_list must be a List of int64, torch.Tensor or None"):
        ops.npu_gmm(x, w, group_list=(4, 8))
    with pytest.raises(TypeError, match="group_list must be a torch.Tensor or None"):
        ops.npu_gmm_v2(x, w, group_list=[4, 4])
    with pytest.raises(ValueError, match="one-dimensional"):
        ops.npu_gmm(x, w, group_list=torch.zeros(2, 2, dtype=torch.int64))
    with pytest.raises(TypeError, match="dtype"):
        ops.npu_gmm(x, w, group_list=torch.zeros(2, dtype=torch.int32))
    with pytest.raises(TypeError, match="group_type"):
        ops.npu_gmm(x, w, group_list=[4, 8], group_type="0")
    with pytest.raises(TypeError, match="non quant"):
        ops.npu_gmm(x, w.to(torch.int8), group_list=[4, 8])
    with pytest.raises(ValueError, match="group_list_type"):
        gmm_mod._npu_gmm_common(None, x, w, group_list=torch.tensor([4, 8]), group_list_type=3)


def test_raw_module_surface():
    # mindspeed/ops/csrc/cann/gmm.cpp:295-309
    mod = ops.GMMFunction.builder.load()
    for name in ("npu_gmm", "npu_gmm_backward", "npu_gmm_backward_fusion"):
        assert callable(getattr(mod, name))
    assert callable(getattr(ops.GMMFunction.builder2.load(), "npu_gmm"))


def test_groupmatmul_add_checks():
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    dy = torch.randn(8, 4, dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="float32"):
        ops.npu_groupmatmul_add_fp32(x, dy, torch.tensor([4, 8]), torch.zeros(32, 4, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="elements"):
        ops.npu_groupmatmul_add_fp32(x, dy, torch.tensor([4, 8]), torch.zeros(31, 4))


def test_routing_map_and_module_api_surface():
    from mindspeed_amd.ops import moe_permute_mask_map as M
    # mindspeed/core/fusions/fused_moe_permute.py:50-57,69-77
    assert list(inspect.signature(M.permute).parameters) == [
        "tokens", "routing_map", "probs", "num_out_tokens", "fused", "drop_and_pad"]
    assert list(inspect.signature(M.unpermute).parameters) == [
        "permuted_tokens", "sorted_indices", "restore_shape", "probs", "routing_map", "fused", "drop_and_pad"]
    # mindspeed/ops/grouped_matmul.py:81
    assert list(inspect.signature(ops.fused_grouped_matmul).parameters) == ["inputs", "m_split", "weights"]
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    rmap = torch.ones(8, 2, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        M.permute(x, rmap)
    with pytest.raises(TypeError, match="should be bool"):
        M.permute(x, rmap.to(torch.int8))
    with pytest.raises(ValueError, match="routing_map is required"):
        M.unpermute(x, torch.zeros(8, dtype=torch.int64), x.shape)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fused_grouped_matmul(x, [4, 4], torch.randn(2, 16, 4, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.MindSpeedTEGroupedLinear(2, 16, 4, params_dtype=torch.bfloat16)(x, [4, 4])
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops._GroupedMatmul.apply(x, torch.randn(2, 16, 4, dtype=torch.bfloat16), torch.zeros(2, 4), [4, 4], 1)


def test_fused_mlp_argument_checks():
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    w1 = torch.randn(2, 16, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.gmm_swiglu(x, w1, torch.tensor([4, 4]))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.grouped_mlp(x, w1, torch.randn(2, 4, 16, dtype=torch.bfloat16), torch.tensor([4, 4]))


def test_megatron_adapter_surface():
    """``Ops`` is what Megatron's ``grouped_gemm_util.ops`` is replaced by
    (mindspeed/core/fusions/grouped_matmul.py:5-21,35-50): same signature and defaults."""
    from mindspeed_amd import fusions

    sig = inspect.signature(fusions.Ops.gmm)
    assert list(sig.parameters) == ["a", "b", "batch_sizes", "trans_b", "gemm_fusion", "original_weight"]
    assert [sig.parameters[n].default for n in ("trans_b", "gemm_fusion", "original_weight")] == [False, False, None]
    assert fusions.grouped_gemm_is_available() is True
    fusions.assert_grouped_gemm_is_available()
    assert fusions.get_device_capability() == (9, 0)
    # mindspeed/core/fusions/fused_moe_permute.py:50-83
    assert list(inspect.signature(fusions.permute).parameters) == [
        "tokens", "routing_map", "probs", "num_out_tokens", "fused", "drop_and_pad"]
    assert list(inspect.signature(fusions.unpermute).parameters) == [
        "permuted_tokens", "sorted_indices", "restore_shape", "probs", "routing_map", "fused", "drop_and_pad"]
    x = torch.randn(8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fusions.Ops.gmm(x, torch.randn(2, 16, 4, dtype=torch.bfloat16), torch.tensor([4, 4]))


def test_shapes_propagate_on_meta_tensors():
    """Every op of the layer carries a fake (meta) kernel, so the Python surface runs on meta tensors, forward and
    backward, without a device: ``torch.ops.mindspeed.npu_gmm`` yields ``(M, N)`` as the reference's Meta
    registration does (mindspeed/op_builder/gmm_builder.py:101-106,141-146)."""
    from mindspeed_amd import fusions
    from mindspeed_amd.dispatcher import dispatch_mlp_combine
    from mindspeed_amd.ops import moe_permute_mask_map as M

    def meta(*shape, dtype=torch.bfloat16, grad=False):
        return torch.empty(*shape, dtype=dtype, device="meta", requires_grad=grad)

    T, H, E, K, F = 64, 32, 4, 2, 48
    x, w = meta(T * K, H, grad=True), meta(E, H, 2 * F, grad=True)
    gl = meta(E, dtype=torch.int64)
    for y in (torch.ops.mindspeed.npu_gmm(None, x, w, group_list=gl),
              torch.ops.mindspeed.npu_gmm(None, x, w, group_list=[32, 64, 96, 128]),
              torch.ops.mindspeed.npu_gmm_v2(None, x, w, group_list=gl),
              ops.npu_gmm(x, w, group_list=gl), fusions.Ops.gmm(x, w, gl)):
        assert y.device.type == "meta" and y.shape == (T * K, 2 * F) and y.dtype == torch.bfloat16
    y.sum().backward()
    assert x.grad.shape == x.shape and w.grad.shape == w.shape
    assert fusions.Ops.gmm(x, meta(E, 2 * F, H), gl, trans_b=True).shape == (T * K, 2 * F)
    dw = ops.npu_gmm(x.detach().t(), meta(T * K, 24), group_list=gl, group_type=2)
    assert dw.shape == (E, H, 24)

    tokens, idx = meta(T, H, grad=True), meta(T, K, dtype=torch.int64)
    permuted, row_map = ops.npu_moe_token_permute(tokens, idx)
    assert permuted.shape == (T * K, H) and row_map.shape == (T * K,) and row_map.dtype == torch.int32
    assert ops.npu_moe_token_permute(tokens, idx, num_out_tokens=100)[0].shape == (100, H)
    probs = meta(T, K, grad=True)
    out = ops.npu_moe_token_unpermute(permuted, row_map, probs)
    assert out.shape == (T, H)
    out.sum().backward()
    assert tokens.grad.shape == (T, H) and probs.grad.shape == (T, K)

    w1, w2 = meta(E, H, 2 * F, grad=True), meta(E, F, H, grad=True)
    out = dispatch_mlp_combine(tokens, idx, probs, (w1, w2))
    assert out.shape == (T, H)
    out.sum().backward()
    assert w1.grad.shape == w1.shape and w2.grad.shape == w2.shape

    rmap, mprobs = meta(T, E, dtype=torch.bool), meta(T, E, dtype=torch.float32, grad=True)
    perm, pp, sidx = M.permute(tokens, rmap, mprobs, num_out_tokens=T * K, fused=True)
    assert perm.shape == (T * K, H) and pp.shape == (T * K,) and sidx.dtype == torch.int64
    assert perm.dtype == torch.bfloat16 and pp.dtype == torch.bfloat16       # the fused hook's dtype rule
    back = M.unpermute(perm, sidx, tokens.shape, probs=mprobs, routing_map=rmap, fused=True)
    assert back.shape == (T, H)
    back.sum().backward()
    assert mprobs.grad.shape == (T, E)

    # the fused matmul + SwiGLU forms, the one-parameter-per-expert module and the chunk sort
    from mindspeed_amd.ops.gmm_swiglu import gmm_swiglu, grouped_mlp
    xs, rp = meta(T * K, H, grad=True), meta(T * K, dtype=torch.float32, grad=True)
    act = gmm_swiglu(xs, w1, gl, rp)
    assert act.shape == (T * K, F) and act.dtype == torch.bfloat16
    act.sum().backward()
    assert xs.grad.shape == xs.shape and rp.grad.shape == rp.shape
    with torch.no_grad():
        assert gmm_swiglu(xs, w1, gl, rp).shape == (T * K, F) and grouped_mlp(xs, w1, w2, gl, rp).shape == (T * K, H)
    for fused in (True, False):
        for recompute in (False, True):
            xm = meta(T * K, H, grad=True)
            out = grouped_mlp(xm, w1, w2, gl, rp, recompute_activation=recompute, fused_kernels=fused)
            assert out.shape == (T * K, H)
            out.sum().backward()
            assert xm.grad.shape == xm.shape
    layer = ops.MindSpeedTEGroupedLinear(E, H, 24, params_dtype=torch.bfloat16, device="meta")
    xl = meta(T * K, H, grad=True)
    yl, bias = layer(xl, [32, 32, 32, 32])
    assert yl.shape == (T * K, 24) and bias is None
    yl.sum().backward()
    assert xl.grad.shape == xl.shape and all(p.grad.shape == (24, H) for p in layer.total_weight)
    xc, pc = meta(T, H, grad=True), meta(T, dtype=torch.float32, grad=True)
    oc, opc = ops.sort_chunks_by_idxs(xc, meta(4, dtype=torch.int64), meta(4, dtype=torch.int64), pc)
    assert oc.shape == (T, H) and opc.shape == (T,)
    (oc.sum() + opc.sum()).backward()
    assert xc.grad.shape == (T, H) and pc.grad.shape == (T,)


def test_caller_side_modules_run_on_meta_tensors():
    """The expert module (one-node and op-by-op bodies, with activation recomputation), ``BF16GMMFunction`` and the fused
    chunk sort's own names carry shapes and gradients on meta tensors: no device is needed to trace them."""
    import types

    import torch.nn.functional as F

    from mindspeed_amd.experts import GroupedMLP
    from mindspeed_amd.grouped_matmul_util import BF16GMMFunction, get_gmm_op_cls
    from mindspeed_amd.ops import sort_chunks as SC

    def meta(*shape, dtype=torch.bfloat16, grad=False):
        return torch.empty(*shape, dtype=dtype, device="meta", requires_grad=grad)

    E, H, FF, R = 4, 64, 32, 100
    tpe = torch.tensor([25, 25, 25, 25])
    for fuse in (True, False):
        for recompute in (False, True):
            cfg = types.SimpleNamespace(hidden_size=H, moe_ffn_hidden_size=FF, gated_linear_unit=True,
                                        activation_func=F.silu, params_dtype=torch.bfloat16, device="meta",
                                        moe_fuse_expert_mlp=fuse, recompute_activation_function=recompute)
            mlp = GroupedMLP(E, cfg)
            mlp.layer_number = 1
            assert mlp.weight1.shape == (H, E * 2 * FF) and mlp.weight2.shape == (E * FF, H)
            x, probs = meta(R, H, grad=True), meta(R, grad=True)
            out, bias = mlp(x, tpe, probs)
            assert out.shape == (R, H) and out.dtype == torch.bfloat16 and bias is None
            out.sum().backward()
            assert x.grad.shape == x.shape and probs.grad.shape == probs.shape
            assert mlp.weight1.grad.shape == mlp.weight1.shape and mlp.weight2.grad.shape == mlp.weight2.shape

    assert get_gmm_op_cls() is BF16GMMFunction
    x, w, gl = meta(R, H, grad=True), meta(E, H, 2 * FF, grad=True), meta(E, dtype=torch.int64)
    y = BF16GMMFunction.apply(x, w, None, gl, 0)
    assert y.shape == (R, 2 * FF)
    y.sum().backward()
    assert x.grad.shape == x.shape and w.grad.shape == w.shape

    with pytest.raises(AssertionError):                  # the fused form takes device tensors only
        SC.moe_sort_chunks_by_index(torch.zeros(8, 4), torch.tensor([4, 4]), torch.tensor([1, 0]))
    xc, pc = meta(R, H, grad=True), meta(R, dtype=torch.float32, grad=True)
    sizes, order = meta(4, dtype=torch.int64), meta(4, dtype=torch.int64)
    assert SC.moe_sort_chunks_by_index(xc, sizes, order).shape == (R, H)
    oc, opc = SC.moe_sort_chunks_by_index_with_probs(xc, pc, sizes, order)
    (oc.sum() + opc.sum()).backward()
    assert xc.grad.shape == (R, H) and pc.grad.shape == (R,)


def test_deferred_weight_gradient_queue_on_meta_tensors():
    """``WeightGradStore`` in decoupled mode: backward returns dX only and parks the weight-gradient operands; ``pop``
    runs the parked product later and adds it to ``main_grad``; ``clear`` resets the switch
    (fb_overlap/modules/weight_grad_store.py:29-58,86-108)."""
    from mindspeed_amd.grouped_matmul_util import BF16GMMFunction, WeightGradStore, gmm_settings

    def meta(*shape, dtype=torch.bfloat16, grad=False):
        return torch.empty(*shape, dtype=dtype, device="meta", requires_grad=grad)

    E, H, N, R = 4, 64, 48, 100
    x, w = meta(R, H, grad=True), torch.nn.Parameter(meta(E, H, N))
    w.main_grad = meta(E, H, N, dtype=torch.float32)
    gl = meta(E, dtype=torch.int64)
    WeightGradStore.clear()
    try:
        WeightGradStore.is_decoupleBlock = True
        y = BF16GMMFunction.apply(x, w, None, gl, w)
        y.sum().backward()
        assert x.grad.shape == x.shape and w.grad is None          # dW was not computed in backward
        assert len(WeightGradStore.cache) == 1
        (ctx_and_inputs, grad_output, weight_param, _sp, _in_row) = WeightGradStore.cache[0]
        assert weight_param is w and grad_output.shape == (R, N) and ctx_and_inputs[1].shape == (R, H)
        for fusion in (False, True):
            gmm_settings.gemm_gradient_accumulation_fusion = fusion
            if fusion:                                                 # park the same operands once more
                WeightGradStore.put(ctx_and_inputs, grad_output, weight_param)
            WeightGradStore.pop()
            assert not WeightGradStore.cache and w.main_grad.shape == (E, H, N)
    finally:
        gmm_settings.gemm_gradient_accumulation_fusion = False
        WeightGradStore.clear()
    assert WeightGradStore.is_decoupleBlock is False and WeightGradStore.cache == []


def test_trace_and_microbench_builds_are_wired():
    """The diagnostic (tile trace) build and the measurement helpers have output paths of their own, and the plain copy
    kernel is not part of the product's C ABI."""
    from mindspeed_amd import _lib, build

    assert build.TRACE_LIB_PATH != build.LIB_PATH and build.TRACE_LIB_PATH.endswith("libmindspeed_amd_trace.so")
    assert build.MICROBENCH_LIB_PATH not in (build.LIB_PATH, build.TRACE_LIB_PATH)
    assert callable(build.build_trace) and callable(build.build_microbench)
    assert not any("copy" in name for name in _lib.EXPORTED_SYMBOLS)
    header = open(os.path.join(os.path.dirname(build.HERE), "include", "mindspeed_amd.h")).read()
    assert "ms_copy_bytes" not in header
