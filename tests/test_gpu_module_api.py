"""GPU parity for the two module-level grouped-matmul APIs (stacked weights with per-group counts, and one
parameter per expert) against the CPU oracle; rel-L2 1e-2 (bf16, fp16) and 1e-5 (fp32)."""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

import mindspeed_amd.ops as ops

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-5}


def say(*a):
    print(*a, flush=True)


CASES = [
    # counts, K, N, dtype
    ([5, 0, 7, 3], 24, 40, torch.float32),
    ([9, 0, 0, 7, 9, 6, 7, 4], 64, 96, torch.bfloat16),        # the reference unit test's group list
    ([130, 256, 1, 300, 64, 0, 200, 73], 256, 512, torch.bfloat16),   # fast path, ragged tails
    ([100, 28], 72, 136, torch.float16),
    ([40, 40, 40], 64, 64, torch.bfloat16),                    # K == N: orientation taken as [E, K, N]
    ([430 + 17 * (i % 5) for i in range(24)], 256, 512, torch.bfloat16),   # many small groups: per-XCD lists
]


def _oracle(x, counts, w_ekn, gy):
    x64 = x.double().requires_grad_(True)
    w64 = w_ekn.double().requires_grad_(True)
    out = O.grouped_matmul(x64, torch.tensor(counts), w64)
    out.backward(gy.double())
    return out, x64.grad, w64.grad


@pytest.mark.parametrize("counts,K,N,dtype", CASES)
@pytest.mark.parametrize("layout", ["EKN", "ENK"])
def test_fused_grouped_matmul(counts, K, N, dtype, layout, device):
    if layout == "ENK" and K == N:
        pytest.skip("square weights are read as [E, K, N] by definition")
    say("stacked-weight case", counts, K, N, dtype, layout)
    E, M = len(counts), sum(counts)
    gen = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, N, generator=gen) * 0.1).to(dtype)
    gy = torch.randn(M, N, generator=gen).to(dtype)
    exp, exp_dx, exp_dw = _oracle(x, counts, w, gy)

    xd = x.to(device).requires_grad_(True)
    stored = w if layout == "EKN" else w.transpose(1, 2).contiguous()
    wd = stored.to(device).requires_grad_(True)
    m_split = torch.tensor(counts, dtype=torch.int64, device=device)
    out = ops.fused_grouped_matmul(xd, m_split, wd)
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == dtype
    assert rel_l2(out, exp) <= TOL[dtype]
    assert rel_l2(xd.grad, exp_dx) <= TOL[dtype]
    dw = wd.grad if layout == "EKN" else wd.grad.transpose(1, 2)
    assert wd.grad.shape == stored.shape
    assert rel_l2(dw, exp_dw) <= TOL[dtype]
    # m_split as a python list goes the same way
    out2 = ops.fused_grouped_matmul(xd.detach(), counts, wd.detach())
    assert torch.equal(out2, out.detach())


@pytest.mark.parametrize("counts,K,N,dtype", CASES)
def test_te_grouped_linear(counts, K, N, dtype, device):
    say("per-expert-parameter case", counts, K, N, dtype)
    E, M = len(counts), sum(counts)
    gen = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, N, generator=gen) * 0.1).to(dtype)
    gy = torch.randn(M, N, generator=gen).to(dtype)
    exp, exp_dx, exp_dw = _oracle(x, counts, w, gy)

    layer = ops.MindSpeedTEGroupedLinear(E, K, N, params_dtype=dtype, device=device)
    with torch.no_grad():
        for i, p in enumerate(layer.total_weight):
            p.copy_(w[i].t())            # parameters are [output_size, input_size]
    xd = x.to(device).requires_grad_(True)
    out, bias = layer(xd, counts)
    assert bias is None
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    assert rel_l2(out, exp) <= TOL[dtype]
    assert rel_l2(xd.grad, exp_dx) <= TOL[dtype]
    for i, p in enumerate(layer.total_weight):
        assert p.grad.shape == (N, K)
        if counts[i] == 0:
            assert torch.count_nonzero(p.grad) == 0
        else:
            assert rel_l2(p.grad.t(), exp_dw[i]) <= TOL[dtype]


def test_stacked_weights_with_bias(device):
    """``_GroupedMatmul`` with per-group bias vectors (the argument that mindspeed/ops/grouped_matmul.py:40-42 passes
    on to the vendor op), as a list and stacked; the bias gets no gradient."""
    counts, K, N, dtype = [130, 0, 300, 77], 64, 96, torch.bfloat16
    say("stacked weights with bias", counts)
    E, M = len(counts), sum(counts)
    gen = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, N, generator=gen) * 0.1).to(dtype)
    bias = torch.randn(E, N, generator=gen).to(dtype)
    exp = O.grouped_matmul(x.double(), counts, w.double()) + torch.repeat_interleave(bias.double(), torch.tensor(counts), dim=0)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    bias_list = [b.to(device) for b in bias]
    out = ops._GroupedMatmul.apply(xd, wd, bias_list, counts, 1)
    out2 = ops._GroupedMatmul.apply(xd, wd, bias.to(device), torch.tensor(counts, device=device), 1)
    assert rel_l2(out, exp) <= TOL[dtype] and torch.equal(out, out2)
    out.sum().backward()
    assert xd.grad.shape == x.shape and wd.grad.shape == w.shape


def test_weight_list_limits(device):
    from mindspeed_amd.ops.gmm import gmm_raw_weight_list
    x = torch.randn(8, 16, device=device)
    ws = [torch.randn(16, 8, device=device) for _ in range(257)]
    counts = torch.zeros(257, dtype=torch.int64, device=device)
    with pytest.raises(Exception, match="outside"):
        gmm_raw_weight_list(x, ws, counts, 1)
    with pytest.raises(ValueError):
        gmm_raw_weight_list(x, [ws[0], torch.randn(16, 9, device=device)], counts[:2], 1)
