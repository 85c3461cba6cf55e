"""GPU parity of the Megatron-facing adapters: ``Ops.gmm`` driven the way Megatron's expert module drives
``grouped_gemm_util.ops`` (mindspeed/core/fusions/grouped_matmul.py:5-21), the zero-token path of the expert
module (mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:154-181), and the layer traced by
``torch.compile`` through the ops' fake kernels."""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

from mindspeed_amd import fusions
from mindspeed_amd.dispatcher import dispatch_mlp_combine
from mindspeed_amd.ops import fused_swiglu, grouped_mlp

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


class FakeGroupedMLP(torch.nn.Module):
    """The calls Megatron's ``GroupedMLP.forward`` makes, with ``gg.ops`` replaced by ``Ops``: weights stored flat
    (``weight1 [H, E*2F]``, ``weight2 [E*F, H]``) and viewed per expert at use (experts.py:90-91)."""

    def __init__(self, E, H, F, dtype, gen):
        super().__init__()
        self.E, self.H, self.F = E, H, F
        self.weight1 = torch.nn.Parameter((torch.randn(H, E * 2 * F, generator=gen) * 0.05).to(dtype))
        self.weight2 = torch.nn.Parameter((torch.randn(E * F, H, generator=gen) * 0.05).to(dtype))

    def forward(self, permuted, tokens_per_expert, gemm_fusion=False):
        w1 = self.weight1.view(self.E, self.H, -1)
        w2 = self.weight2.view(self.E, -1, self.H)
        if permuted.nelement() != 0:
            fc1 = fusions.Ops.gmm(permuted, w1, tokens_per_expert, trans_b=False, gemm_fusion=gemm_fusion,
                                  original_weight=self.weight1)
            act = fused_swiglu(fc1)
            return fusions.Ops.gmm(act, w2, tokens_per_expert, trans_b=False, gemm_fusion=gemm_fusion,
                                   original_weight=self.weight2)
        # no tokens on this rank: plain matmuls on the flat weights, so the parameters still get (zero) gradients
        assert torch.count_nonzero(tokens_per_expert) == 0
        h = torch.matmul(permuted, self.weight1.view(self.H, -1))
        h = torch.nn.functional.silu(h[..., : h.size(-1) // 2]) * h[..., h.size(-1) // 2:]
        return torch.matmul(h, self.weight2.view(-1, self.H))


@pytest.mark.parametrize("where", ["device", "host"])
def test_ops_gmm_with_a_megatron_style_caller(where, device):
    """Forward and all gradients of the expert module against the oracle; ``tokens_per_expert`` on the device or on
    the host, as Megatron keeps it."""
    say("Ops.gmm caller, batch sizes on", where)
    gen = torch.Generator().manual_seed(31)
    E, H, F, dtype = 6, 128, 96, torch.bfloat16
    counts = torch.tensor([70, 0, 300, 5, 129, 64])
    M = int(counts.sum())
    mlp = FakeGroupedMLP(E, H, F, dtype, gen).to(device)
    x = torch.randn(M, H, generator=gen).to(dtype)
    gy = torch.randn(M, H, generator=gen).to(dtype)
    xd = x.to(device).requires_grad_(True)
    tpe = counts.to(device) if where == "device" else counts
    out = mlp(xd, tpe)
    out.backward(gy.to(device))
    torch.cuda.synchronize()

    x_ref = x.clone().requires_grad_(True)
    w1 = mlp.weight1.detach().cpu().view(E, H, -1).clone().requires_grad_(True)
    w2 = mlp.weight2.detach().cpu().view(E, -1, H).clone().requires_grad_(True)
    exp = O.experts_computation(x_ref, counts, w1, w2)
    exp.backward(gy)
    assert rel_l2(out, exp) <= 1e-2
    assert rel_l2(xd.grad, x_ref.grad) <= 2e-2
    assert rel_l2(mlp.weight1.grad.view(E, H, -1), w1.grad) <= 2e-2
    assert rel_l2(mlp.weight2.grad.view(E, -1, H), w2.grad) <= 2e-2
    assert torch.count_nonzero(mlp.weight1.grad.view(E, H, -1)[1]) == 0          # the expert without rows

    # trans_b: the same weights stored transposed per expert and read through a strided view
    w1t = mlp.weight1.detach().view(E, H, -1).transpose(1, 2).contiguous()
    y_t = fusions.Ops.gmm(xd.detach(), w1t, tpe, trans_b=True)
    y_n = fusions.Ops.gmm(xd.detach(), mlp.weight1.detach().view(E, H, -1), tpe)
    assert torch.equal(y_t, y_n)


def test_ops_gmm_gemm_fusion_accumulates_into_main_grad(device):
    gen = torch.Generator().manual_seed(32)
    E, H, F, dtype = 4, 64, 48, torch.bfloat16
    counts = torch.tensor([33, 0, 200, 23])
    M = int(counts.sum())
    mlp = FakeGroupedMLP(E, H, F, dtype, gen).to(device)
    for p in (mlp.weight1, mlp.weight2):
        p.main_grad = torch.zeros(p.shape, dtype=torch.float32, device=device)
        p.grad_added_to_main_grad = False
    x = torch.randn(M, H, generator=gen).to(dtype)
    gy = torch.randn(M, H, generator=gen).to(dtype)
    out = mlp(x.to(device).requires_grad_(True), counts.to(device), gemm_fusion=True)
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    w1 = mlp.weight1.detach().cpu().view(E, H, -1).clone().requires_grad_(True)
    w2 = mlp.weight2.detach().cpu().view(E, -1, H).clone().requires_grad_(True)
    O.experts_computation(x, counts, w1, w2).backward(gy)
    assert mlp.weight1.grad_added_to_main_grad and mlp.weight2.grad_added_to_main_grad
    assert rel_l2(mlp.weight1.main_grad.view(E, H, -1), w1.grad) <= 2e-2
    assert rel_l2(mlp.weight2.main_grad.view(E, -1, H), w2.grad) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_zero_tokens_give_zero_weight_gradients(dtype, device):
    """A rank that received no tokens: every op runs on zero rows, the outputs are empty and the weights get
    all-zero gradients of their own shape (the reference reaches the same through its plain-matmul branch,
    experts.py:154-181)."""
    say("zero-token case", dtype)
    gen = torch.Generator().manual_seed(33)
    E, H, F = 4, 64, 48
    counts = torch.zeros(E, dtype=torch.int64, device=device)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.05).to(dtype).to(device).requires_grad_(True)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.05).to(dtype).to(device).requires_grad_(True)
    x = torch.empty(0, H, dtype=dtype, device=device, requires_grad=True)
    # the op sequence of the expert module on the grouped-matmul kernels
    fc1 = fusions.Ops.gmm(x, w1, counts)
    out = fusions.Ops.gmm(fused_swiglu(fc1), w2, counts)
    assert fc1.shape == (0, 2 * F) and out.shape == (0, H)
    out.backward(torch.empty(0, H, dtype=dtype, device=device))
    torch.cuda.synchronize()
    assert x.grad.shape == (0, H)
    for w in (w1, w2):
        assert w.grad is not None and w.grad.shape == w.shape and torch.count_nonzero(w.grad) == 0
    # the fused expert MLP (one autograd node) on the same empty input
    if dtype != torch.float32:
        w1.grad = w2.grad = None
        out = grouped_mlp(x, w1, w2, counts)
        assert out.shape == (0, H)
        out.backward(torch.empty(0, H, dtype=dtype, device=device))
        torch.cuda.synchronize()
        for w in (w1, w2):
            assert w.grad.shape == w.shape and torch.count_nonzero(w.grad) == 0
    # the reference's own branch for this case on the flat weights: also zero gradients, same shapes
    mlp = FakeGroupedMLP(E, H, F, dtype, gen).to(device)
    mlp(x.detach().requires_grad_(True), counts).backward(torch.empty(0, H, dtype=dtype, device=device))
    assert torch.count_nonzero(mlp.weight1.grad) == 0 and torch.count_nonzero(mlp.weight2.grad) == 0


@pytest.mark.parametrize("fuse", [False, True])
def test_layer_traced_by_torch_compile(fuse, device):
    """``torch.compile`` (AOT-traced, eager kernels) of the whole layer, forward and backward, with one kernel per op
    and with the SwiGLU passes fused into the grouped matmuls: the trace goes through the ops' fake kernels, the run
    through the same HIP kernels, so results equal the eager ones bit for bit."""
    gen = torch.Generator().manual_seed(34)
    T, H, E, K, F, dtype = 256, 128, 8, 2, 96, torch.bfloat16
    x = torch.randn(T, H, generator=gen).to(dtype).to(device)
    p, idx = O.route_topk(torch.randn(T, E, generator=gen), K)
    p, idx = p.to(dtype).to(device), idx.to(device)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.05).to(dtype).to(device)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.05).to(dtype).to(device)
    gy = torch.randn(T, H, generator=gen).to(dtype).to(device)

    def layer(x, p, w1, w2):
        return dispatch_mlp_combine(x, idx, p, (w1, w2), fuse_activation=fuse)

    def run(fn):
        leaves = [t.clone().requires_grad_(True) for t in (x, p, w1, w2)]
        out = fn(*leaves)
        return (out.detach(), *torch.autograd.grad(out, leaves, gy))

    eager = run(layer)
    compiled = run(torch.compile(layer, backend="aot_eager"))
    torch.cuda.synchronize()
    for name, a, b in zip(("out", "dx", "dprobs", "dw1", "dw2"), eager, compiled):
        assert torch.equal(a, b), name
