"""GPU parity of the grouped matmul with the SwiGLU activation fused into its epilogue: against the CPU
oracle (rel-L2 1e-2) and, bit for bit, against the two separate kernels it replaces."""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

import mindspeed_amd.ops as ops
from mindspeed_amd.dispatcher import dispatch_mlp_combine, experts_computation

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


CASES = [
    # counts, K, ffn, dtype, probs dtype (None = no probs), rows past the last offset
    ([5, 0, 7, 3], 64, 128, torch.bfloat16, torch.float32, 0),
    ([9, 0, 0, 7, 9, 6, 7, 4], 128, 200, torch.bfloat16, None, 0),          # ffn not a multiple of 128
    ([130, 256, 1, 300, 64, 0, 200, 73], 256, 384, torch.bfloat16, torch.bfloat16, 5),   # 64-/128-row tails
    ([300, 212], 72, 136, torch.float16, torch.float32, 0),
    ([1024, 1000, 1048], 512, 1024, torch.bfloat16, torch.float32, 0),       # full tiles, many rounds
    ([40], 8, 8, torch.bfloat16, torch.float32, 0),                          # smallest legal sizes
    # many small groups with enough tiles for several rounds: whole groups go to single XCDs (per-XCD lists)
    ([520 + 13 * (i % 7) for i in range(32)], 256, 768, torch.bfloat16, torch.float32, 9),
]


@pytest.mark.parametrize("counts,K,ffn,dtype,pdt,extra", CASES)
def test_gmm_swiglu_forward_backward(counts, K, ffn, dtype, pdt, extra, device):
    say("gmm_swiglu case", counts, K, ffn, dtype, pdt, extra)
    E, M = len(counts), sum(counts) + extra
    gen = torch.Generator().manual_seed(M + ffn)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, 2 * ffn, generator=gen) * 0.1).to(dtype)
    probs = None if pdt is None else (torch.rand(M, generator=gen) + 0.25).to(pdt)
    g_act = torch.randn(M, ffn, generator=gen).to(dtype)
    gl = torch.tensor(counts, dtype=torch.int64)

    # the two separate kernels
    xs = x.to(device).requires_grad_(True)
    ws = w.to(device).requires_grad_(True)
    ps = None if probs is None else probs.to(device).requires_grad_(True)
    fc1 = ops.npu_gmm_v2(xs, ws, group_list=gl.to(device), group_type=0)
    act_sep = ops.swiglu_with_probs(fc1, ps) if ps is not None else ops.fused_swiglu(fc1)
    act_sep.backward(g_act.to(device))

    # fused
    xf = x.to(device).requires_grad_(True)
    wf = w.to(device).requires_grad_(True)
    pf = None if probs is None else probs.to(device).requires_grad_(True)
    act = ops.gmm_swiglu(xf, wf, gl.to(device), pf)
    act.backward(g_act.to(device))
    torch.cuda.synchronize()
    assert act.shape == (M, ffn) and act.dtype == dtype
    assert torch.equal(act, act_sep)                       # same values, bit for bit
    assert torch.equal(xf.grad, xs.grad) and torch.equal(wf.grad, ws.grad)
    if probs is not None:
        assert torch.equal(pf.grad, ps.grad)

    # oracle (fc1 rounded to the storage dtype before the activation, as the op sequence does)
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    p64 = None if probs is None else probs.double().requires_grad_(True)
    fc1_o = O.gmm(x64, w64, gl, group_type=0, group_list_type=1)
    act_o = O.swiglu(fc1_o, p64)
    act_o.backward(g_act.double())
    assert rel_l2(act, act_o) <= 1e-2
    assert rel_l2(xf.grad, x64.grad) <= 1e-2
    assert rel_l2(wf.grad, w64.grad) <= 1e-2
    if probs is not None:
        assert rel_l2(pf.grad, p64.grad) <= 1e-2
    if extra:
        assert torch.count_nonzero(act[M - extra:]) == 0   # rows past the last offset


def test_layer_uses_the_fused_kernel_and_matches_the_unfused_layer(device):
    T, H, E, K, F = 300, 128, 8, 2, 256
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(T, H, generator=gen).to(torch.bfloat16).to(device)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.05).to(torch.bfloat16).to(device)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.05).to(torch.bfloat16).to(device)
    p, idx = O.route_topk(torch.randn(T, E, generator=gen), K)
    p, idx = p.to(torch.bfloat16).to(device), idx.to(device)
    from mindspeed_amd import flop_counter
    with flop_counter.record(timing=False) as rec:
        out = dispatch_mlp_combine(x, idx, p, (w1, w2), fuse_activation=True)
    names = [c[0] for c in rec.calls]
    assert "swiglu" not in names and "gmm_fwd_swiglu" in names        # activation came out of the first matmul
    perm, rmap, _, counts = ops.moe_token_permute_with_aux(x, idx, num_experts=E)
    ref = ops.npu_moe_token_unpermute(experts_computation(perm, counts, w1, w2, fuse_activation=False), rmap, p)
    assert torch.equal(out, ref)


def test_unsupported_layout_is_reported(device):
    x = torch.randn(16, 12, device=device).to(torch.bfloat16)            # K not a multiple of 8
    w = torch.randn(2, 12, 32, device=device).to(torch.bfloat16)
    gl = torch.tensor([8, 8], dtype=torch.int64, device=device)
    with pytest.raises(Exception, match="vector-access"):
        ops.gmm_swiglu(x, w, gl)
    with pytest.raises(TypeError):
        ops.gmm_swiglu(x.float(), w.float(), gl)


MLP_CASES = [
    # counts, K (hidden), ffn, dtype, probs dtype, rows past the last offset
    ([5, 0, 7, 3], 64, 128, torch.bfloat16, torch.float32, 0),
    ([9, 0, 0, 7, 9, 6, 7, 4], 128, 200, torch.bfloat16, None, 0),
    ([130, 256, 1, 300, 64, 0, 200, 73], 256, 384, torch.bfloat16, torch.bfloat16, 5),
    ([300, 212], 72, 136, torch.float16, torch.float32, 0),
    ([700, 1000, 348], 512, 1024, torch.bfloat16, torch.float32, 0),
    # many small groups: per-XCD lists in the fused kernels, forward and backward
    ([430 + 17 * (i % 5) for i in range(24)], 256, 512, torch.bfloat16, torch.float32, 6),
]


@pytest.mark.parametrize("counts,K,ffn,dtype,pdt,extra", MLP_CASES)
@pytest.mark.parametrize("recompute", [False, True])
@pytest.mark.parametrize("fused_kernels", [True, False])
def test_grouped_mlp_forward_backward(counts, K, ffn, dtype, pdt, extra, recompute, fused_kernels, device):
    _grouped_mlp_case(counts, K, ffn, dtype, pdt, extra, recompute, fused_kernels, device)


# layouts and dtypes only the one-kernel-per-op node takes: fp32, and sizes that rule out 16-byte accesses
UNFUSED_ONLY_CASES = [
    ([5, 0, 7, 3], 64, 96, torch.float32, torch.float32, 0),
    ([33, 20, 0, 11], 36, 50, torch.bfloat16, torch.float32, 3),
    ([17, 40], 30, 27, torch.float16, None, 0),
]


@pytest.mark.parametrize("counts,K,ffn,dtype,pdt,extra", UNFUSED_ONLY_CASES)
def test_grouped_mlp_separate_kernels_any_layout(counts, K, ffn, dtype, pdt, extra, device):
    _grouped_mlp_case(counts, K, ffn, dtype, pdt, extra, False, False, device)


def _grouped_mlp_case(counts, K, ffn, dtype, pdt, extra, recompute, fused_kernels, device):
    say("grouped_mlp case", counts, K, ffn, dtype, pdt, extra, recompute, fused_kernels)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    E, M = len(counts), sum(counts) + extra
    gen = torch.Generator().manual_seed(M + ffn + 1)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w1 = (torch.randn(E, K, 2 * ffn, generator=gen) * 0.1).to(dtype)
    w2 = (torch.randn(E, ffn, K, generator=gen) * 0.1).to(dtype)
    probs = None if pdt is None else (torch.rand(M, generator=gen) + 0.25).to(pdt)
    gy = torch.randn(M, K, generator=gen).to(dtype)
    gl = torch.tensor(counts, dtype=torch.int64)

    def leaves():
        out = [t.to(device).requires_grad_(True) for t in (x, w1, w2)]
        out.append(None if probs is None else probs.to(device).requires_grad_(True))
        return out

    # the separate kernels
    xs, w1s, w2s, ps = leaves()
    fc1 = ops.npu_gmm_v2(xs, w1s, group_list=gl.to(device), group_type=0)
    act = ops.swiglu_with_probs(fc1, ps) if ps is not None else ops.fused_swiglu(fc1)
    out_sep = ops.npu_gmm_v2(act, w2s, group_list=gl.to(device), group_type=0)
    out_sep.backward(gy.to(device))

    xf, w1f, w2f, pf = leaves()
    out = ops.grouped_mlp(xf, w1f, w2f, gl.to(device), pf, recompute_activation=recompute,
                          fused_kernels=fused_kernels)
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    assert torch.equal(out, out_sep)
    assert torch.equal(xf.grad, xs.grad)                   # d_fc1 is bit-identical, so everything behind it is
    assert torch.equal(w1f.grad, w1s.grad) and torch.equal(w2f.grad, w2s.grad)
    if probs is not None and fused_kernels:
        # same terms, summed per 64 columns and then over the row instead of in one pass
        assert rel_l2(pf.grad, ps.grad) <= (1e-5 if pdt == torch.float32 else 1e-2)
    elif probs is not None:
        assert torch.equal(pf.grad, ps.grad)               # the very same kernel

    x64, w164, w264 = (t.double().requires_grad_(True) for t in (x, w1, w2))
    p64 = None if probs is None else probs.double().requires_grad_(True)
    fc1_o = O.gmm(x64, w164, gl, group_type=0, group_list_type=1)
    out_o = O.gmm(O.swiglu(fc1_o, p64), w264, gl, group_type=0, group_list_type=1)
    out_o.backward(gy.double())
    assert rel_l2(out, out_o) <= tol
    assert rel_l2(xf.grad, x64.grad) <= tol
    assert rel_l2(w1f.grad, w164.grad) <= tol and rel_l2(w2f.grad, w264.grad) <= tol
    if probs is not None:
        assert rel_l2(pf.grad, p64.grad) <= tol


def test_inference_skips_the_fc1_output(device):
    """Under ``torch.no_grad()`` the fused forward does not store the fc1 output (the kernel's NULL-output form):
    the activation and the MLP output are bit for bit those of the differentiable call."""
    say("fused forward without fc1 output")
    counts, K, ffn, dtype = [130, 256, 1, 300, 64, 0, 200, 73], 256, 384, torch.bfloat16
    M, E = sum(counts) + 5, len(counts)
    gen = torch.Generator().manual_seed(23)
    x = torch.randn(M, K, generator=gen).to(dtype).to(device)
    w1 = (torch.randn(E, K, 2 * ffn, generator=gen) * 0.05).to(dtype).to(device)
    w2 = (torch.randn(E, ffn, K, generator=gen) * 0.05).to(dtype).to(device)
    probs = torch.rand(M, generator=gen).to(device)
    gl = torch.tensor(counts, dtype=torch.int64, device=device)
    act = ops.gmm_swiglu(x.clone().requires_grad_(True), w1, gl, probs)
    out = ops.grouped_mlp(x.clone().requires_grad_(True), w1, w2, gl, probs)
    before = torch.cuda.memory_allocated(device)
    with torch.no_grad():
        act_inf = ops.gmm_swiglu(x, w1, gl, probs)
        assert torch.cuda.memory_allocated(device) - before < 2 * act_inf.numel() * act_inf.element_size() + (1 << 20)
        out_inf = ops.grouped_mlp(x, w1, w2, gl, probs)
    torch.cuda.synchronize()
    assert torch.equal(act_inf, act.detach()) and torch.equal(out_inf, out.detach())
    # real parameters (requires_grad) under no_grad: still the inference form.  (Inside the autograd function the
    # inputs' requires_grad is visible whatever the grad mode, so the decision is taken before it.)
    w1p, w2p = torch.nn.Parameter(w1), torch.nn.Parameter(w2)
    fc1_bytes = M * 2 * ffn * x.element_size()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(device)
    before = torch.cuda.memory_allocated(device)
    with torch.no_grad():
        out_p = ops.grouped_mlp(x, w1p, w2p, gl, probs)
    torch.cuda.synchronize()
    # peak = activation + output + tile table (1.3 MB here); with the fc1 output (1.6 MB) beside the activation it
    # would be at least 2.4 MB
    assert torch.cuda.max_memory_allocated(device) - before < fc1_bytes + (1 << 18)
    torch.cuda.reset_peak_memory_stats(device)
    before = torch.cuda.memory_allocated(device)
    with torch.no_grad():
        act_p = ops.gmm_swiglu(x, w1p, gl, probs)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated(device) - before < fc1_bytes       # the activation alone is half of it
    assert not act_p.requires_grad and not out_p.requires_grad
    assert torch.equal(act_p, act.detach()) and torch.equal(out_p, out.detach())
    # and with grad mode on the same parameters get their gradients
    out_t = ops.grouped_mlp(x, w1p, w2p, gl, probs)
    out_t.sum().backward()
    assert w1p.grad is not None and w2p.grad is not None and torch.equal(out_t.detach(), out.detach())


def test_layer_default_under_no_grad_is_the_fused_form(device):
    """``dispatch_mlp_combine`` without a ``fuse_activation`` argument: one kernel per op where gradients may follow,
    the fused form under ``torch.no_grad()``; both give the same bits."""
    say("layer default under no_grad")
    from mindspeed_amd import flop_counter
    T, H, E, K, F, dtype = 512, 256, 8, 2, 384, torch.bfloat16
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(T, H, generator=gen).to(dtype).to(device)
    p, idx = O.route_topk(torch.randn(T, E, generator=gen), K)
    p, idx = p.to(dtype).to(device), idx.to(device)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.05).to(dtype).to(device)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.05).to(dtype).to(device)
    with flop_counter.record(timing=False) as rec:
        with_grad = dispatch_mlp_combine(x.clone().requires_grad_(True), idx, p, (w1, w2))
    assert "swiglu" in rec.summary() and "gmm_fwd_swiglu" not in rec.summary()
    with torch.no_grad(), flop_counter.record(timing=False) as rec:
        inference = dispatch_mlp_combine(x, idx, p, (w1, w2))
        separate = dispatch_mlp_combine(x, idx, p, (w1, w2), fuse_activation=False)
    assert "gmm_fwd_swiglu" in rec.summary()
    assert torch.equal(inference, with_grad.detach()) and torch.equal(inference, separate)
