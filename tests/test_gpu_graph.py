"""GPU: the whole single-rank expert layer (forward and backward; with and without the weight-gradient products
on a second stream) recorded into a HIP graph and replayed.  Every replay, with eager work of the same ops and
synchronisations in between, must reproduce the eager result bit for bit: the C ABI only launches kernels on
the caller's stream (no allocation, no synchronisation, no memset node), which is what makes it capturable."""
import pytest
import torch

from mindspeed_amd.dispatcher import dispatch_mlp_combine

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def make_inputs(T, H, E, K, F, dtype, device, seed):
    gen = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(T, H, generator=gen, device=device).to(dtype)
    logits = torch.randn(T, E, generator=gen, device=device)
    probs, idx = torch.topk(torch.softmax(logits, dim=-1), K, dim=-1)
    probs = (probs / probs.sum(-1, keepdim=True)).to(dtype)
    w1 = (torch.randn(E, H, 2 * F, generator=gen, device=device) * 0.05).to(dtype)
    w2 = (torch.randn(E, F, H, generator=gen, device=device) * 0.05).to(dtype)
    gy = torch.randn(T, H, generator=gen, device=device).to(dtype)
    return x, idx, probs, w1, w2, gy


def layer_step(x, idx, probs, w1, w2, gy, fuse):
    x = x.detach().requires_grad_(True)
    probs = probs.detach().requires_grad_(True)
    w1 = w1.detach().requires_grad_(True)
    w2 = w2.detach().requires_grad_(True)
    out = dispatch_mlp_combine(x, idx, probs, (w1, w2), fuse_activation=fuse)
    grads = torch.autograd.grad(out, (x, probs, w1, w2), gy)
    return (out,) + tuple(grads)


@pytest.mark.parametrize("overlap", [False, True])
@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("T,H,E,K,F", [(512, 256, 8, 2, 512), (300, 128, 6, 3, 200)])
def test_layer_graph_replays_match_eager(T, H, E, K, F, fuse, overlap, device, monkeypatch):
    say("graph case", T, H, E, K, F, fuse, overlap)
    import mindspeed_amd.ops.gmm as gmm_ops
    monkeypatch.setattr(gmm_ops, "OVERLAP_WGRAD", overlap)     # weight gradients beside dX on a second stream, or after
    dtype = torch.bfloat16
    a = make_inputs(T, H, E, K, F, dtype, device, seed=1)
    b = make_inputs(T, H, E, K, F, dtype, device, seed=2)
    eager_a = [t.clone() for t in layer_step(*a, fuse)]     # also the warm-up that precedes any capture
    eager_b = [t.clone() for t in layer_step(*b, fuse)]
    torch.cuda.synchronize()

    static = [t.clone() for t in a]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph):
            outs = layer_step(*static, fuse)
    torch.cuda.current_stream(device).wait_stream(side)
    torch.cuda.synchronize()

    for rep, (src, want) in enumerate([(a, eager_a), (b, eager_b), (a, eager_a), (b, eager_b)]):
        for dst, s in zip(static, src):
            dst.copy_(s)
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip(outs, want):
            assert torch.equal(got, exp), f"replay {rep} differs from the eager result"
        # eager work of the same ops between replays
        again = layer_step(*src, fuse)
        torch.cuda.synchronize()
        for got, exp in zip(again, want):
            assert torch.equal(got, exp)
