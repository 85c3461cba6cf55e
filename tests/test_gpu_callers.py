"""GPU parity of the caller-side classes and names the reference reaches the kernels through:

* the expert module ``GmmExpertsImpl`` / ``GroupedMLP`` (mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:14-193)
  in all its branches: op by op, as one fused node, with ``gemm_gradient_accumulation_fusion``, with activation
  recomputation (``CheckpointWithoutOutput``), and with no tokens on the rank;
* ``BF16GMMFunction`` with its separable ``op_forward / op_dx / op_dw / op_gmm_add`` and the deferred weight gradient
  of the forward/backward-overlap schedules (grouped_matmul_util.py:41-184, weight_grad_store.py:86-108);
* the fused chunk sort's own names (mindspeed/lite/ops/triton/sort_chunks_by_idx.py:67-115,167-221,300-348);
* ``permute`` / ``unpermute`` / ``fused_permute`` / ``fused_unpermute`` of the expert-parallel dispatcher
  (mindspeed/fsdp/distributed/expert_parallel/utils.py:10-69).

Everything is compared with the CPU oracle (rel-L2 <= 1e-2 for bf16 outputs, 2e-2 for bf16 gradients; integer maps
and row movement exactly)."""
import types

import pytest
import torch
import torch.nn.functional as F

from conftest import rel_l2
from oracle import moe_oracle as O

from mindspeed_amd import expert_parallel_utils as ep
from mindspeed_amd import grouped_matmul_util as gu
from mindspeed_amd.experts import GroupedMLP
from mindspeed_amd.ops import sort_chunks as sc
from mindspeed_amd.recompute import CheckpointWithoutOutput

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _config(H, ffn, dtype, device, **kw):
    cfg = types.SimpleNamespace(hidden_size=H, moe_ffn_hidden_size=ffn, gated_linear_unit=True, activation_func=F.silu,
                                params_dtype=dtype, device=device, gemm_gradient_accumulation_fusion=False,
                                recompute_activation_function=False)
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


def _oracle_mlp(module, x, counts, probs, gy, E, H):
    x_ref = x.clone().requires_grad_(True)
    w1 = module.weight1.detach().cpu().view(E, H, -1).clone().requires_grad_(True)
    w2 = module.weight2.detach().cpu().view(E, -1, H).clone().requires_grad_(True)
    p_ref = probs.clone().requires_grad_(True) if probs is not None else None
    fc1 = O.gmm(x_ref, w1, counts, 0, 1)
    act = O.swiglu(fc1, p_ref)
    out = O.gmm(act, w2, counts, 0, 1)
    out.backward(gy)
    return out, x_ref.grad, w1.grad, w2.grad, (p_ref.grad if p_ref is not None else None)


@pytest.mark.parametrize("mode", ["one_node", "op_by_op", "recompute_one_node", "recompute_op_by_op"])
def test_expert_module_against_oracle(mode, device):
    say("expert module", mode)
    gen = torch.Generator().manual_seed(41)
    E, H, ffn, dtype = 6, 128, 96, torch.bfloat16
    counts = torch.tensor([70, 0, 300, 5, 129, 64])
    M = int(counts.sum())
    cfg = _config(H, ffn, dtype, device, moe_fuse_expert_mlp=mode.endswith("one_node"),
                  recompute_activation_function=mode.startswith("recompute"))
    torch.manual_seed(7)
    mlp = GroupedMLP(E, cfg)
    mlp.layer_number = 1
    assert mlp.weight1.shape == (H, E * 2 * ffn) and mlp.weight2.shape == (E * ffn, H) and mlp.weight1.is_cuda
    x = torch.randn(M, H, generator=gen).to(dtype)
    probs = torch.rand(M, generator=gen).to(dtype)
    gy = torch.randn(M, H, generator=gen).to(dtype)
    xd = x.to(device).requires_grad_(True)
    pd = probs.to(device).requires_grad_(True)
    out, bias = mlp(xd, counts.to(device), pd)
    assert bias is None and out.shape == (M, H)
    if mode == "recompute_op_by_op":
        # the activation's storage is released between forward and backward
        assert mlp.activation_checkpoint_manager.outputs[0].untyped_storage().size() == 0
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    exp, dx, dw1, dw2, dp = _oracle_mlp(mlp, x, counts, probs, gy, E, H)
    assert rel_l2(out, exp) <= 1e-2
    assert rel_l2(xd.grad, dx) <= 2e-2
    assert rel_l2(mlp.weight1.grad.view(E, H, -1), dw1) <= 2e-2
    assert rel_l2(mlp.weight2.grad.view(E, -1, H), dw2) <= 2e-2
    assert rel_l2(pd.grad, dp) <= 2e-2
    assert torch.count_nonzero(mlp.weight1.grad.view(E, H, -1)[1]) == 0          # the expert without rows


def test_expert_module_modes_agree_bit_for_bit(device):
    """One fused node, the reference's op sequence, and both with activation recomputation: same output and same
    gradients, bit for bit (the fused kernels compute from the rounded fc1 values exactly what the separate ones do)."""
    gen = torch.Generator().manual_seed(42)
    E, H, ffn, dtype = 4, 256, 128, torch.bfloat16
    counts = torch.tensor([200, 56, 0, 300])
    M = int(counts.sum())
    x = torch.randn(M, H, generator=gen).to(dtype).to(device)
    probs = torch.rand(M, generator=gen).to(dtype).to(device)
    gy = torch.randn(M, H, generator=gen).to(dtype).to(device)
    results = []
    for fuse in (True, False):
        for recompute in (False, True):
            cfg = _config(H, ffn, dtype, device, moe_fuse_expert_mlp=fuse, recompute_activation_function=recompute)
            torch.manual_seed(9)
            mlp = GroupedMLP(E, cfg)
            mlp.layer_number = 3
            xd = x.clone().requires_grad_(True)
            out, _ = mlp(xd, counts.to(device), probs)
            out.backward(gy)
            results.append((out.detach(), xd.grad, mlp.weight1.grad, mlp.weight2.grad))
    torch.cuda.synchronize()
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b)


def test_expert_module_gemm_fusion_and_zero_tokens(device):
    gen = torch.Generator().manual_seed(43)
    E, H, ffn, dtype = 4, 64, 48, torch.bfloat16
    counts = torch.tensor([33, 0, 200, 23])
    M = int(counts.sum())
    cfg = _config(H, ffn, dtype, device, gemm_gradient_accumulation_fusion=True)
    mlp = GroupedMLP(E, cfg)
    for p in (mlp.weight1, mlp.weight2):
        p.main_grad = torch.zeros(p.shape, dtype=torch.float32, device=device)
        p.grad_added_to_main_grad = False
    x = torch.randn(M, H, generator=gen).to(dtype)
    probs = torch.rand(M, generator=gen).to(dtype)
    gy = torch.randn(M, H, generator=gen).to(dtype)
    out, _ = mlp(x.to(device).requires_grad_(True), counts, probs.to(device))       # tokens_per_expert on the host
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    exp, _, dw1, dw2, _ = _oracle_mlp(mlp, x, counts, probs, gy, E, H)
    assert rel_l2(out, exp) <= 1e-2
    assert mlp.weight1.grad_added_to_main_grad and mlp.weight2.grad_added_to_main_grad
    assert rel_l2(mlp.weight1.main_grad.view(E, H, -1), dw1) <= 2e-2
    assert rel_l2(mlp.weight2.main_grad.view(E, -1, H), dw2) <= 2e-2
    # no tokens on the rank: empty output, all-zero gradients of the parameters' own shapes (experts.py:154-181)
    for recompute in (False, True):
        cfg0 = _config(H, ffn, dtype, device, recompute_activation_function=recompute)
        mlp0 = GroupedMLP(E, cfg0)
        mlp0.layer_number = 1
        x0 = torch.empty(0, H, dtype=dtype, device=device, requires_grad=True)
        out0, _ = mlp0(x0, torch.zeros(E, dtype=torch.int64, device=device), torch.empty(0, dtype=dtype, device=device))
        assert out0.shape == (0, H)
        out0.backward(torch.empty(0, H, dtype=dtype, device=device))
        for w in (mlp0.weight1, mlp0.weight2):
            assert w.grad is not None and w.grad.shape == w.shape and torch.count_nonzero(w.grad) == 0


def test_checkpoint_without_output_on_the_activation(device):
    """The helper by itself: output storage released, rebuilt by the hook, gradients equal to the plain graph's."""
    gen = torch.Generator().manual_seed(44)
    a = torch.randn(64, 32, generator=gen).to(device).requires_grad_(True)
    b = torch.randn(64, 1, generator=gen).to(device).requires_grad_(True)
    w = torch.randn(16, 8, generator=gen).to(device).requires_grad_(True)
    fn = lambda x, p: (F.silu(x[:, :16]) * x[:, 16:] * p)             # noqa: E731
    ref = (fn(a, b) @ w)
    ga, gb, gw = torch.autograd.grad(ref.sum(), (a, b, w))
    mgr = CheckpointWithoutOutput()
    act = mgr.checkpoint(fn, False, a, b)
    y = act @ w
    mgr.discard_output()
    assert act.untyped_storage().size() == 0
    y.register_hook(mgr.recompute)
    y.sum().backward()
    assert torch.equal(a.grad, ga) and torch.equal(b.grad, gb) and torch.equal(w.grad, gw)
    with pytest.raises(RuntimeError, match="distribute_saved_activations"):
        CheckpointWithoutOutput().checkpoint(fn, True, a, b)


# ---- BF16GMMFunction ---------------------------------------------------------------------------------------------------
def _gmm_problem(device, seed=51):
    gen = torch.Generator().manual_seed(seed)
    E, H, N, dtype = 5, 96, 160, torch.bfloat16
    counts = [64, 0, 130, 7, 255]
    M = sum(counts)
    x = torch.randn(M, H, generator=gen).to(dtype)
    w = (torch.randn(E, H, N, generator=gen) * 0.05).to(dtype)
    gy = torch.randn(M, N, generator=gen).to(dtype)
    exp_y = O.gmm(x, w, torch.tensor(counts), 0, 1)
    exp_dx, exp_dw = O.gmm_backward(gy, x, w, torch.tensor(counts), 1)
    return E, H, N, counts, x, w, gy, exp_y, exp_dx, exp_dw


def test_bf16_gmm_function_products_and_autograd(device):
    E, H, N, counts, x, w, gy, exp_y, exp_dx, exp_dw = _gmm_problem(device)
    cls = gu.get_gmm_op_cls()
    assert cls is gu.BF16GMMFunction and gu.get_gmm_quant_func() is None
    xd, wd, gyd = x.to(device), w.to(device), gy.to(device)
    cum = torch.cumsum(torch.tensor(counts), 0).to(device)
    # the three products by themselves, list in / list out
    (y,) = cls.op_forward(None, xd, wd, cum)
    (dx,) = cls.op_dx(None, gyd, wd, cum)
    (dw,) = cls.op_dw(None, xd, gyd, cum)
    torch.cuda.synchronize()
    assert rel_l2(y, exp_y) <= 1e-2 and rel_l2(dx, exp_dx) <= 1e-2
    assert dw.shape == (E, H, N) and rel_l2(dw, exp_dw) <= 1e-2 and torch.count_nonzero(dw[1]) == 0
    # as an autograd node: gmm_apply takes tokens per expert (a list or a tensor) and the parameter object
    param = torch.nn.Parameter(wd.clone())
    xr = xd.clone().requires_grad_(True)
    out = cls.gmm_apply(xr, param, None, counts, param)
    out.backward(gyd)
    torch.cuda.synchronize()
    assert torch.equal(out.detach(), y)
    assert torch.equal(xr.grad, dx) and torch.equal(param.grad, dw)


def test_deferred_weight_gradient_runs_later_detached_from_dx(device):
    """``WeightGradStore.is_decoupleBlock``: backward returns dX only and parks the operands; ``pop()`` later runs the
    K-grouped matmul by itself — as a plain product added to ``main_grad``, or (gemm fusion) accumulated in place."""
    E, H, N, counts, x, w, gy, exp_y, exp_dx, exp_dw = _gmm_problem(device, seed=52)
    cls = gu.BF16GMMFunction
    xd, gyd = x.to(device), gy.to(device)
    try:
        for fusion in (False, True):
            say("deferred dW, gemm fusion", fusion)
            gu.WeightGradStore.clear()
            gu.gmm_settings.gemm_gradient_accumulation_fusion = fusion
            param = torch.nn.Parameter(w.to(device))
            param.main_grad = torch.full((E * H, N), 0.5, dtype=torch.float32, device=device)
            param.grad_added_to_main_grad = False
            xr = xd.clone().requires_grad_(True)
            out = cls.gmm_apply(xr, param.view(E, H, N), None, torch.tensor(counts, device=device), param)
            gu.WeightGradStore.is_decoupleBlock = True
            out.backward(gyd)
            torch.cuda.synchronize()
            assert rel_l2(xr.grad, exp_dx) <= 1e-2
            assert param.grad is None and len(gu.WeightGradStore.cache) == 1
            assert torch.all(param.main_grad == 0.5)                       # nothing has touched it yet
            gu.WeightGradStore.is_decoupleBlock = False
            gu.WeightGradStore.pop()
            torch.cuda.synchronize()
            assert not gu.WeightGradStore.cache
            assert rel_l2(param.main_grad.view(E, H, N) - 0.5, exp_dw) <= 1e-2
            assert torch.all(param.main_grad.view(E, H, N)[1] == 0.5)       # empty expert: += 0
    finally:
        gu.WeightGradStore.clear()
        gu.gmm_settings.gemm_gradient_accumulation_fusion = False


def test_gmm_function_gemm_fusion_in_backward(device):
    E, H, N, counts, x, w, gy, exp_y, exp_dx, exp_dw = _gmm_problem(device, seed=53)
    try:
        gu.gmm_settings.gemm_gradient_accumulation_fusion = True
        param = torch.nn.Parameter(w.to(device))
        param.main_grad = torch.zeros(E * H, N, dtype=torch.float32, device=device)
        param.grad_added_to_main_grad = False
        xr = x.to(device).requires_grad_(True)
        out = gu.BF16GMMFunction.gmm_apply(xr, param.view(E, H, N), None, counts, param)
        out.backward(gy.to(device))
        torch.cuda.synchronize()
        assert param.grad_added_to_main_grad
        assert rel_l2(param.main_grad.view(E, H, N), exp_dw) <= 1e-2 and rel_l2(xr.grad, exp_dx) <= 1e-2
    finally:
        gu.gmm_settings.gemm_gradient_accumulation_fusion = False


# ---- the fused chunk sort's names ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("num_splits,num_tokens,hidden", [(16, 2048, 256), (32, 4096, 128), (6, 100, 24)])
def test_chunk_sort_names(num_splits, num_tokens, hidden, device):
    """The reference test's sizes (tests_extend/.../test_sort_chunks_by_idx.py:250-253) and a ragged odd one."""
    gen = torch.Generator().manual_seed(num_splits)
    cuts = torch.sort(torch.randint(0, num_tokens + 1, (num_splits - 1,), generator=gen))[0]
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([num_tokens])]))
    order = torch.randperm(num_splits, generator=gen)
    inp = torch.randn(num_tokens, hidden, generator=gen).to(torch.bfloat16)
    probs = torch.rand(num_tokens, generator=gen)
    exp, exp_p = O.sort_chunks_by_idxs(inp, sizes.tolist(), order.tolist(), probs)
    # brute-force map: output row of every source row
    starts = torch.cat([torch.tensor([0]), torch.cumsum(sizes, 0)])
    dst = 0
    exp_map = torch.full((num_tokens,), -1, dtype=torch.int32)
    for c in order.tolist():
        n = int(sizes[c])
        exp_map[int(starts[c]):int(starts[c]) + n] = torch.arange(dst, dst + n, dtype=torch.int32)
        dst += n
    sd, od, xd, pd = sizes.to(device), order.to(device), inp.to(device), probs.to(device)
    row_id_map = sc.make_chunk_sort_map(sd, od, num_tokens, num_splits)
    assert row_id_map.dtype == torch.int32 and torch.equal(row_id_map.cpu(), exp_map)
    fwd, fwd_p = sc.sort_chunks_by_map(xd, row_id_map, pd, num_tokens, hidden, is_forward=True)
    assert torch.equal(fwd.cpu(), exp) and torch.equal(fwd_p.cpu(), exp_p)
    back, back_p = sc.sort_chunks_by_map(fwd, row_id_map, fwd_p, num_tokens, hidden, is_forward=False)
    assert torch.equal(back, xd) and torch.equal(back_p, pd)
    only, none = sc.sort_chunks_by_map(xd, row_id_map, None, num_tokens, hidden, is_forward=True)
    assert none is None and torch.equal(only, fwd)
    # the differentiable wrappers
    xr = xd.clone().requires_grad_(True)
    pr = pd.clone().requires_grad_(True)
    out = sc.moe_sort_chunks_by_index(xr, sd, od)
    assert torch.equal(out.detach().cpu(), exp)
    out2, out_p = sc.moe_sort_chunks_by_index_with_probs(xr, pr, sd, od)
    assert torch.equal(out2.detach().cpu(), exp) and torch.equal(out_p.detach().cpu(), exp_p)
    gy = torch.randn(num_tokens, hidden, generator=gen).to(torch.bfloat16).to(device)
    gp = torch.rand(num_tokens, generator=gen).to(device)
    torch.autograd.backward([out2, out_p], [gy, gp])
    # the backward is the inverse movement
    assert torch.equal(xr.grad, sc.sort_chunks_by_map(gy, row_id_map, None, num_tokens, hidden, False)[0])
    assert torch.equal(pr.grad, sc.sort_chunks_by_map(gy, row_id_map, gp, num_tokens, hidden, False)[1])
    with pytest.raises(AssertionError):
        sc.moe_sort_chunks_by_index(xd, sizes, od)          # host tensor: the fused form takes device tensors only
    empty = torch.empty(0, hidden, dtype=torch.bfloat16, device=device)
    assert sc.moe_sort_chunks_by_index(empty, sd, od) is empty


# ---- permute / unpermute of the expert-parallel dispatcher ------------------------------------------------------------------
@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("topk", [1, 2, 8])
def test_expert_parallel_permute_unpermute(topk, idx_dtype, device):
    gen = torch.Generator().manual_seed(60 + topk)
    T, H, E, dtype = 300, 128, 16, torch.bfloat16
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    probs_full, idx = O.route_topk(torch.randn(T, E, generator=gen), topk)
    idx = idx.to(idx_dtype)
    if topk == 1:
        idx = idx.view(-1)
    probs = probs_full.to(dtype)
    td, idd, pd = tokens.to(device), idx.to(device), probs.to(device)
    exp_perm, exp_sorted = O.permute(tokens, idx)
    exp_out = O.unpermute(exp_perm, exp_sorted, probs if topk > 1 else None)
    # eager convention: forward order, in the indices' dtype
    perm, sorted_indices = ep.permute(td, idd, fused=False)
    assert sorted_indices.dtype == idx_dtype
    assert torch.equal(perm.cpu(), exp_perm) and torch.equal(sorted_indices.cpu().long(), exp_sorted.long())
    out = ep.unpermute(perm, sorted_indices, pd if topk > 1 else None, fused=False)
    assert rel_l2(out, exp_out) <= 1e-2
    # fused convention: the int32 row map
    perm_f, row_map = ep.permute(td, idd, fused=True)
    assert row_map.dtype == torch.int32 and torch.equal(perm_f, perm)
    assert torch.equal(row_map.cpu().long(), O.row_id_map(idx).long())
    out_f = ep.unpermute(perm_f, row_map, pd if topk > 1 else None, fused=True)
    assert torch.equal(out_f, out)
    with pytest.raises(AssertionError):
        ep.unpermute(perm_f[:-1], row_map, None, fused=True)
    # fp32 probabilities: the fused form casts the rows to the probabilities' dtype first (utils.py:37-38)
    if topk > 1:
        out32 = ep.fused_unpermute(perm_f, row_map, pd.float())
        assert out32.dtype == torch.float32
        assert rel_l2(out32, O.unpermute(exp_perm.float(), exp_sorted, probs.float())) <= 1e-5
    if topk > 1:
        i2, w2 = ep.normalize_expert_args(pd, idd)             # swapped on purpose
        assert i2 is idd and w2 is pd
    if topk > 1 and idx_dtype == torch.int64:
        full = torch.rand(T, E, generator=gen).to(device)
        _, g = ep.normalize_expert_args(idd, full)
        assert torch.equal(g, full.gather(1, idd))
