"""GPU parity: SwiGLU, chunk sort and the whole single-rank expert layer
(permute -> gmm -> silu*gate -> gmm -> weighted unpermute) against the CPU
oracle and the fp64 golden fixture."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

import mindspeed_amd.ops as ops
from mindspeed_amd.dispatcher import dispatch_mlp_combine

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-5}


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,ffn", [(1024, 512), (333, 1408), (50, 37)])
def test_swiglu(rows, ffn, dtype, device):
    say("swiglu", rows, ffn, dtype)
    gen = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, 2 * ffn, generator=gen).to(dtype)
    p = torch.rand(rows, generator=gen).to(dtype)
    gy = torch.randn(rows, ffn, generator=gen).to(dtype)
    tol = TOL[dtype]
    xd = x.to(device).requires_grad_(True)
    y = ops.fused_swiglu(xd)
    y.backward(gy.to(device))
    assert rel_l2(y, O.swiglu(x.double())) <= tol
    ex, _ = O.swiglu_backward(gy, x)
    assert rel_l2(xd.grad, ex) <= tol
    xd2 = x.to(device).requires_grad_(True)
    pd = p.to(device).requires_grad_(True)
    y2 = ops.swiglu_with_probs(xd2, pd)
    y2.backward(gy.to(device))
    assert rel_l2(y2, O.swiglu(x.double(), p.double())) <= tol
    ex2, ep2 = O.swiglu_backward(gy, x, p)
    assert rel_l2(xd2.grad, ex2) <= tol and rel_l2(pd.grad, ep2) <= tol


@pytest.mark.parametrize("nchunks,rows,hidden", [(16, 2048, 256), (32, 4096, 128), (5, 77, 10)])
def test_sort_chunks(nchunks, rows, hidden, device):
    say("sort_chunks", nchunks, rows, hidden)
    gen = torch.Generator().manual_seed(nchunks)
    cuts = torch.sort(torch.randint(0, rows + 1, (nchunks - 1,), generator=gen))[0]
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([rows])]))
    order = torch.randperm(nchunks, generator=gen)
    x = torch.randn(rows, hidden, generator=gen)
    p = torch.rand(rows, generator=gen)
    eo, ep = O.sort_chunks_by_idxs(x, sizes, order, p)
    xd = x.to(device).requires_grad_(True)
    out, outp = ops.sort_chunks_by_idxs(xd, sizes.to(device), order.to(device), p.to(device))
    assert torch.equal(out.cpu(), eo) and torch.equal(outp.cpu(), ep)          # a pure row copy: exact
    g = torch.randn(rows, hidden, generator=gen)
    out.backward(g.to(device))
    exp_g = torch.empty_like(g)
    starts = torch.cat([torch.tensor([0]), torch.cumsum(sizes, 0)])
    src_rows = torch.cat([torch.arange(starts[i], starts[i] + sizes[i]) for i in order.tolist()])
    exp_g[src_rows] = g
    assert torch.equal(xd.grad.cpu(), exp_g)
    out2, none = ops.sort_chunks_by_idxs(x.to(device), sizes.tolist(), order.tolist())
    assert none is None and torch.equal(out2.cpu(), eo)


def test_sort_chunks_partial_map_on_the_device(device):
    """Sizes and order given as device tensors cannot be checked without a read-back: rows that a partial map leaves
    out (sizes summing to less than the row count, a chunk named twice and another never) read as zeros, forward
    and backward, instead of uninitialised memory."""
    say("sort_chunks partial map")
    gen = torch.Generator().manual_seed(5)
    rows, hidden = 1000, 64
    x = torch.randn(rows, hidden, generator=gen)
    p = torch.rand(rows, generator=gen)
    poison = torch.full((1 << 22,), float("nan"), device=device)       # whatever the allocator hands out next is NaN
    del poison
    # 1. the sizes cover 900 of the 1000 rows
    sizes = torch.tensor([300, 100, 500]); order = torch.tensor([2, 0, 1])
    xd = x.to(device).requires_grad_(True)
    out, outp = ops.sort_chunks_by_idxs(xd, sizes.to(device), order.to(device), p.to(device))
    want = torch.cat([x[400:900], x[0:300], x[300:400], torch.zeros(100, hidden)])
    assert torch.equal(out.cpu(), want)
    assert torch.equal(outp.cpu(), torch.cat([p[400:900], p[0:300], p[300:400], torch.zeros(100)]))
    g = torch.randn(rows, hidden, generator=gen)
    out.backward(g.to(device))
    exp_g = torch.zeros(rows, hidden)
    exp_g[400:900], exp_g[0:300], exp_g[300:400] = g[0:500], g[500:800], g[800:900]
    assert torch.equal(xd.grad.cpu(), exp_g)
    # 2. chunk 0 named twice, chunk 1 never: 600 output rows are written, the input rows of chunk 1 get no gradient
    sizes = torch.tensor([300, 700]); order = torch.tensor([0, 0])
    xd = x.to(device).requires_grad_(True)
    out, _ = ops.sort_chunks_by_idxs(xd, sizes.to(device), order.to(device))
    assert torch.equal(out.cpu(), torch.cat([x[0:300], x[0:300], torch.zeros(400, hidden)]))
    out.backward(g.to(device))
    got = xd.grad.cpu()
    assert not torch.isnan(got).any() and torch.equal(got[300:], torch.zeros(700, hidden))


@pytest.mark.parametrize("dtype,pdt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32),
                                       (torch.float32, torch.float32)])
@pytest.mark.parametrize("nchunks,rows,hidden", [(64, 8192, 512), (1500, 6000, 24), (2600, 40000, 8), (7, 300, 13)])
def test_sort_chunks_sizes_and_dtypes(nchunks, rows, hidden, dtype, pdt, device):
    """Many chunks (more than one scan pass), empty chunks, every dtype and the element path; a pure row copy,
    so every output is exact.  Chunk counts follow experts x ranks of the reference's dispatcher
    (mindspeed/core/transformer/moe/moe_feature/overlap/moe_common.py:377-398)."""
    say("sort_chunks case", nchunks, rows, hidden, dtype, pdt)
    gen = torch.Generator().manual_seed(nchunks + rows)
    cuts = torch.sort(torch.randint(0, rows + 1, (nchunks - 1,), generator=gen))[0]
    cuts[: nchunks // 4] = cuts[nchunks // 4]                 # a run of empty chunks at the front
    sizes = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([rows])]))
    order = torch.randperm(nchunks, generator=gen)
    x = torch.randn(rows, hidden, generator=gen).to(dtype)
    p = torch.rand(rows, generator=gen).to(pdt)
    eo, ep = O.sort_chunks_by_idxs(x, sizes, order, p)
    xd = x.to(device).requires_grad_(True)
    pd = p.to(device).requires_grad_(True)
    out, outp = ops.sort_chunks_by_idxs(xd, sizes.to(device), order.to(device), pd)
    assert torch.equal(out.cpu(), eo) and torch.equal(outp.cpu(), ep)
    g = torch.randn(rows, hidden, generator=gen).to(dtype)
    gp = torch.rand(rows, generator=gen).to(pdt)
    torch.autograd.backward((out, outp), (g.to(device), gp.to(device)))
    starts = torch.cat([torch.tensor([0]), torch.cumsum(sizes, 0)])
    src_rows = torch.cat([torch.arange(starts[i], starts[i] + sizes[i]) for i in order.tolist()])
    exp_g, exp_gp = torch.empty_like(g), torch.empty_like(gp)
    exp_g[src_rows] = g
    exp_gp[src_rows] = gp
    assert torch.equal(xd.grad.cpu(), exp_g) and torch.equal(pd.grad.cpu(), exp_gp)


def test_layer_fp64_fixture(device):
    g = np.load(os.path.join(GOLDEN, "layer_fp64.npz"))
    x, idx, p = (torch.from_numpy(g[k]).to(device) for k in ("x", "idx", "p"))
    w1, w2 = torch.from_numpy(g["w1"]).to(device), torch.from_numpy(g["w2"]).to(device)
    out = dispatch_mlp_combine(x, idx, p, (w1, w2))
    assert rel_l2(out, torch.from_numpy(g["out"])) <= 1e-5


def _plumbing_inputs(dtype):
    torch.manual_seed(0)
    T, H, E, K, F = 512, 256, 8, 2, 512
    x = torch.randn(T, H)
    p, idx = O.route_topk(torch.randn(T, E), K)
    w1 = torch.randn(E, H, 2 * F) * 0.02
    w2 = torch.randn(E, F, H) * 0.02
    return x.to(dtype), idx, p.to(dtype), w1.to(dtype), w2.to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plumbing_config_forward_backward(dtype, device):
    """512 tokens, hidden 256, 8 experts, top-2, FFN 512, seed 0: forward and all gradients vs the oracle."""
    say("plumbing config", dtype)
    x, idx, p, w1, w2 = _plumbing_inputs(dtype)
    leaves = [t.clone().requires_grad_(True) for t in (x, p, w1, w2)]
    exp = O.moe_layer(leaves[0], idx, leaves[1], leaves[2], leaves[3])
    gy = torch.randn(exp.shape, generator=torch.Generator().manual_seed(1)).to(dtype)
    exp_grads = torch.autograd.grad(exp, leaves, gy)

    dl = [t.to(device).requires_grad_(True) for t in (x, p, w1, w2)]
    out = dispatch_mlp_combine(dl[0], idx.to(device), dl[1], (dl[2], dl[3]))
    out.backward(gy.to(device))
    tol = TOL[dtype]
    assert rel_l2(out, exp) <= tol
    # gradients pass through two rounded GEMMs; bf16 intermediate rounding differs between the paths
    gtol = tol if dtype == torch.float32 else 2e-2
    for name, got, want in zip(("dx", "dprobs", "dw1", "dw2"), (t.grad for t in dl), exp_grads):
        assert rel_l2(got, want) <= gtol, name


def test_mixtral_shape_sampled_tokens(device):
    """Full Mixtral-shape layer (4096 tokens, hidden 4096, 8 experts, top-2, FFN 14336, bf16): sampled tokens
    against a per-token fp32 evaluation, and the combine's linearity in the probabilities."""
    say("mixtral layer sampled")
    T, H, E, K, F = 4096, 4096, 8, 2, 14336
    gen = torch.Generator(device=device).manual_seed(0)
    x = torch.randn(T, H, generator=gen, device=device).to(torch.bfloat16)
    w1 = (torch.randn(E, H, 2 * F, generator=gen, device=device) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(E, F, H, generator=gen, device=device) * 0.02).to(torch.bfloat16)
    p, idx = O.route_topk(torch.randn(T, E, generator=torch.Generator().manual_seed(0)), K)
    p = p.to(torch.bfloat16).to(device)
    idx = idx.to(device)
    out = dispatch_mlp_combine(x, idx, p, (w1, w2))
    assert torch.equal(dispatch_mlp_combine(x, idx, p * 0.5, (w1, w2)), out * 0.5)   # exact scaling by 1/2
    for t in torch.randint(0, T, (24,), generator=torch.Generator().manual_seed(2)).tolist():
        ref = torch.zeros(H, dtype=torch.float32)
        for j in range(K):
            e = int(idx[t, j])
            h = (x[t].float() @ w1[e].float()).to(torch.bfloat16).float()
            a = (torch.nn.functional.silu(h[:F]) * h[F:]).to(torch.bfloat16).float()
            ref += p[t, j].float().cpu() * (a @ w2[e].float()).to(torch.bfloat16).float().cpu()
        assert rel_l2(out[t], ref) <= 1e-2, t


@pytest.mark.parametrize("fuse", [False, True])
def test_weight_gradients_beside_dx_give_identical_results(fuse, device, monkeypatch):
    """The optional second stream for the weight-gradient products (MINDSPEED_AMD_OVERLAP_WGRAD=1) changes when the
    kernels run, not what they compute: every output and gradient of the layer is bit-equal to the default order."""
    say("layer with and without the dX / dW overlap", fuse)
    import mindspeed_amd.ops.gmm as gmm_ops
    gen = torch.Generator().manual_seed(3)
    T, H, E, K, F = 1500, 512, 8, 2, 768
    x = torch.randn(T, H, generator=gen).to(torch.bfloat16).to(device)
    probs, idx = torch.topk(torch.softmax(torch.randn(T, E, generator=gen), dim=-1), K, dim=-1)
    probs, idx = probs.to(torch.bfloat16).to(device), idx.to(device)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.05).to(torch.bfloat16).to(device)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.05).to(torch.bfloat16).to(device)
    gy = torch.randn(T, H, generator=gen).to(torch.bfloat16).to(device)
    results = []
    for overlap in (False, True, False):
        monkeypatch.setattr(gmm_ops, "OVERLAP_WGRAD", overlap)
        leaves = [t.detach().clone().requires_grad_(True) for t in (x, probs, w1, w2)]
        out = dispatch_mlp_combine(leaves[0], idx, leaves[1], (leaves[2], leaves[3]), fuse_activation=fuse)
        grads = torch.autograd.grad(out, leaves, gy)
        torch.cuda.synchronize()
        results.append((out,) + tuple(grads))
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b)
