"""GPU: the reference's own test and documentation flows for the grouped matmul, replayed at their own sizes through
the same entry points (the raw builder module, ``npu_groupmatmul_add_fp32``, ``npu_gmm`` / ``npu_gmm_v2``), with the
reference's own tolerances where it states them."""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

from mindspeed_amd.ops import gmm
from mindspeed_amd.ops.gmm import GMMFunction
from mindspeed_amd.ops.npu_groupmatmul_add import npu_groupmatmul_add_fp32

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype,m,k,n,offsets", [
    (torch.float16, 1024, 4096, 2048, [500, 1024]),                 # test_groupmatmul_add.py:16-33
    (torch.bfloat16, 8192, 8192, 2048, [1024, 2048, 4096, 8192]),   # test_groupmatmul_add.py:39-55
])
def test_groupmatmul_add_as_the_reference_tests_it(dtype, m, k, n, offsets, device):
    """``out + dw`` from the separate weight-gradient op against the fused in-place add, uniform [0, 1) operands,
    ``allclose(rtol=0.005, atol=0.005)`` (tests_extend/unit_tests/ops/atb/test_groupmatmul_add.py:16-33,39-55; the
    reference skips both cases on its current version)."""
    say("groupmatmul_add reference flow", dtype, m, k, n, offsets)
    gen = torch.Generator().manual_seed(k + n)
    e = len(offsets)
    x = torch.rand((m, k), generator=gen).to(dtype).to(device)
    grads_out = torch.rand((m, n), generator=gen).to(dtype).to(device)
    group_list = torch.tensor(offsets, dtype=torch.int64, device=device)
    out = torch.rand((e * k, n), generator=gen).to(device)
    weight = torch.rand((e, k, n), generator=gen).to(dtype).to(device)

    _, dy, _ = GMMFunction.builder.load().npu_gmm_backward([grads_out], [x], [weight], group_list, 0)
    out_single = out + dy[0].view(*out.shape)

    fused = out.clone().detach()
    npu_groupmatmul_add_fp32(x.clone().detach(), grads_out.clone().detach(), group_list.clone().detach(), fused)
    assert torch.allclose(out_single, fused, rtol=0.005, atol=0.005)
    # and against the oracle, which the rounding of the separate op's 16-bit result does not touch
    exp = O.groupmatmul_add_fp32(x.cpu(), grads_out.cpu(), offsets, out.cpu().clone())
    assert rel_l2(fused, exp) <= 1e-5


def test_documented_calls(device):
    """The calls of docs/zh/ops/gmm.md: cumulative list and counts tensor, fp16, 32 rows x 256 over 8 experts,
    forward and backward with a gradient of ones, and the transposed-weight call.  The documentation's counts
    example [1, 3, 3, 4, 5, 6, 7, 4] adds up to 33 for its 32 rows: what the vendor kernel makes of the surplus row
    is not stated anywhere in the reference; here the last group ends where the rows end."""
    num_expert, seq_len, hidden_dim = 8, 32, 256
    dtype = torch.float16
    gen = torch.Generator().manual_seed(0)
    x = (torch.rand((seq_len, hidden_dim), generator=gen).to(dtype) - 0.5)
    weight = (torch.rand((num_expert, hidden_dim, seq_len), generator=gen).to(dtype) - 0.5)
    weight_trans = (torch.rand((num_expert, seq_len, hidden_dim), generator=gen).to(dtype) - 0.5)
    cases = [("npu_gmm", [1, 3, 6, 10, 15, 21, 28, 32], [1, 2, 3, 4, 5, 6, 7, 4]),
             ("npu_gmm_v2", torch.tensor([1, 3, 3, 4, 5, 6, 7, 4]), [1, 3, 3, 4, 5, 6, 7, 3])]
    for name, group_list, counts in cases:
        say("documented call", name)
        fn = getattr(gmm, name)
        gl = group_list.to(device) if torch.is_tensor(group_list) else group_list
        xd = x.to(device).requires_grad_(True)
        wd = weight.to(device).requires_grad_(True)
        result = fn(xd, wd, bias=None, group_list=gl, group_type=0)
        result.backward(torch.ones(result.shape, dtype=dtype, device=device))
        x64 = x.double().requires_grad_(True)
        w64 = weight.double().requires_grad_(True)
        exp = O.grouped_matmul(x64, counts, w64)
        exp.backward(torch.ones_like(exp))
        assert result.shape == (seq_len, seq_len)
        assert rel_l2(result, exp) <= 1e-2 and rel_l2(xd.grad, x64.grad) <= 1e-2 and rel_l2(wd.grad, w64.grad) <= 1e-2
        # weight stored transposed, passed as a view
        wt = weight_trans.to(device).requires_grad_(True)
        result_t = fn(xd.detach(), wt.transpose(-1, -2), bias=None, group_list=gl, group_type=0)
        exp_t = O.grouped_matmul(x.double(), counts, weight_trans.double().transpose(-1, -2))
        assert rel_l2(result_t, exp_t) <= 1e-2


def _per_expert_products(x, weight, group_list, group_type):
    """The comparison the reference's unit test builds: split, one ``@`` per expert, concatenated
    (tests_extend/unit_tests/ops/cann/test_npu_gmm.py:36-50)."""
    if group_type == 0:
        xs, ws = list(x.split(group_list, dim=0)), list(weight)
    else:
        xs, ws = list(x.split(group_list, dim=-1)), list(weight.split(group_list, dim=0))
    return torch.cat([h @ w for h, w in zip(xs, ws)], dim=0)


@pytest.mark.parametrize("mode", ["list_cumsum", "tensor_cumsum", "tensor_count"])
def test_npu_gmm_as_the_reference_tests_it(mode, device):
    """tests_extend/unit_tests/ops/cann/test_npu_gmm.py:57-96 (split on rows) and :100-128 (split on the reduction
    dim, with two empty groups): fp16 normal operands, ``allclose(rtol=0.005, atol=0.005)`` against per-expert
    products."""
    say("npu_gmm reference flow", mode)
    gen = torch.Generator().manual_seed(5)
    dtype = torch.float16
    # split on rows
    weight = torch.randn(8, 64, 32, generator=gen).to(dtype).to(device)
    if mode == "tensor_count":
        x = torch.randn(42, 64, generator=gen).to(dtype).to(device)
        counts = [1, 3, 5, 7, 9, 6, 7, 4]
        y = gmm.npu_gmm_v2(x, weight, bias=None, group_list=torch.tensor(counts, dtype=torch.int64, device=device), group_type=0)
    else:
        x = torch.randn(32, 64, generator=gen).to(dtype).to(device)
        counts = [1, 2, 3, 4, 5, 6, 7, 4]
        cum = [1, 3, 6, 10, 15, 21, 28, 32]
        gl = cum if mode == "list_cumsum" else torch.tensor(cum, dtype=torch.int64, device=device)
        y = gmm.npu_gmm(x, weight, bias=None, group_list=gl, group_type=0)
    assert torch.allclose(y, _per_expert_products(x, weight, counts, 0), rtol=0.005, atol=0.005)
    # split on the reduction dim
    if mode == "tensor_count":
        weight2 = torch.randn(42, 64, generator=gen).to(dtype).to(device)
        x2 = torch.randn(42, 48, generator=gen).to(dtype).to(device).transpose(-1, -2)
        counts = [9, 0, 0, 7, 9, 6, 7, 4]
        y2 = gmm.npu_gmm_v2(x2, weight2, bias=None, group_list=torch.tensor(counts, dtype=torch.int64, device=device), group_type=2)
    else:
        weight2 = torch.randn(32, 64, generator=gen).to(dtype).to(device)
        x2 = torch.randn(32, 48, generator=gen).to(dtype).to(device).transpose(-1, -2)
        counts = [1, 2, 3, 4, 5, 6, 7, 4]
        cum = [1, 3, 6, 10, 15, 21, 28, 32]
        gl = cum if mode == "list_cumsum" else torch.tensor(cum, dtype=torch.int64, device=device)
        y2 = gmm.npu_gmm(x2, weight2, bias=None, group_list=gl, group_type=2)
    assert torch.allclose(y2.reshape(-1, 64), _per_expert_products(x2, weight2, counts, 2), rtol=0.005, atol=0.005)
