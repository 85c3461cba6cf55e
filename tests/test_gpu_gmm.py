"""GPU parity: grouped matmul forward, dX, dW and the fp32 accumulate form
against the CPU oracle and the integer golden fixtures, through the Python
surface that calls the C ABI.  Tolerance: rel-L2 <= 1e-2 for bf16 / fp16,
<= 1e-5 for fp32; integer-valued fixtures must match exactly."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

import mindspeed_amd.ops as ops
from mindspeed_amd.ops.gmm import gmm_raw

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-5}
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reference_test_shapes_exact(dtype, device):
    """Shapes / group lists of the reference's own unit test, on integers: exact in every dtype."""
    g = np.load(os.path.join(GOLDEN, "gmm_cases.npz"))
    for name in ("rows_a", "rows_b", "rows_doc"):
        say("golden", name, dtype)
        counts = g[f"{name}_counts"].tolist()
        x = torch.from_numpy(g[f"{name}_x"]).to(dtype).to(device)
        w = torch.from_numpy(g[f"{name}_w"]).to(dtype).to(device)
        y = torch.from_numpy(g[f"{name}_y"]).float()
        cum = np.cumsum(counts).tolist()
        assert torch.equal(ops.npu_gmm(x, w, bias=None, group_list=cum, group_type=0).float().cpu(), y)
        assert torch.equal(ops.npu_gmm(x, w, group_list=torch.tensor(cum, device=device), group_type=0).float().cpu(), y)
        assert torch.equal(ops.npu_gmm_v2(x, w, group_list=torch.tensor(counts, device=device), group_type=0).float().cpu(), y)
    for name in ("red_a", "red_empty"):
        say("golden", name, dtype)
        counts = g[f"{name}_counts"].tolist()
        x = torch.from_numpy(g[f"{name}_x"]).to(dtype).to(device)      # [M, 48]; the op sees x.T
        w = torch.from_numpy(g[f"{name}_w"]).to(dtype).to(device)
        y = torch.from_numpy(g[f"{name}_y"]).float()
        got = ops.npu_gmm_v2(x.t(), w, group_list=torch.tensor(counts, device=device), group_type=2)
        assert got.shape == y.shape and torch.equal(got.float().cpu(), y)
        got = ops.npu_gmm(x.t(), w, group_list=np.cumsum(counts).tolist(), group_type=2)
        assert torch.equal(got.float().cpu(), y)


def test_groupmatmul_add_fixture(device):
    g = np.load(os.path.join(GOLDEN, "groupmatmul_add.npz"))
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        say("groupmatmul_add golden", dtype)
        x = torch.from_numpy(g["x"]).to(dtype).to(device)
        dy = torch.from_numpy(g["dy"]).to(dtype).to(device)
        acc = torch.from_numpy(g["acc"]).float().to(device)
        ops.npu_groupmatmul_add_fp32(x, dy, torch.from_numpy(g["offsets"]).to(device), acc)
        assert torch.equal(acc.cpu(), torch.from_numpy(g["expect"]).float())


def _counts(kind, E, M, seed):
    gen = torch.Generator().manual_seed(seed)
    if kind == "equal":
        c = torch.full((E,), M // E)
        c[-1] += M - c.sum()
    elif kind == "skew_empty":                     # Zipf-like skew with one empty group
        w = 1.0 / torch.arange(1, E + 1).float() ** 1.2
        w = w[torch.randperm(E, generator=gen)]
        w[int(torch.randint(0, E, (1,), generator=gen))] = 0
        c = torch.floor(w / w.sum() * M).long()
        c[int(torch.argmax(c))] += M - c.sum()
    else:                                          # random, several empty
        cuts = torch.sort(torch.randint(0, M + 1, (E - 1,), generator=gen))[0]
        c = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([M])]))
    assert c.sum() == M and (c >= 0).all()
    return c.long()


GMM_CASES = [
    # M, K, N, E, kind
    (1024, 256, 1024, 8, "random"),
    (1000, 200, 328, 8, "random"),        # nothing a multiple of the tile
    (513, 72, 40, 3, "skew_empty"),
    (4096, 512, 768, 8, "skew_empty"),
    (2048, 128, 512, 64, "random"),       # many small groups, several < 64 rows
    (300, 64, 256, 1, "equal"),
    (96, 1000, 24, 4, "equal"),           # long reduction, narrow output
    (37, 19, 23, 5, "random"),            # tiny and odd: element-wise paths
    (96, 20, 16, 3, "random"),            # dX writes 20 columns: a multiple of 4 but not of 8
    (256, 72, 44, 2, "equal"),            # forward writes 44 columns (n % 8 == 4) from vector-aligned operands
    # tile order in 4 x 8 blocks with partly filled blocks on both sides: 6 / 7 row tiles and 9 column panels in
    # forward, 6 x 9 in the weight gradient; 11 row tiles x 17 column panels (4 + 4 + 3, 8 + 8 + 1) in the last one
    (3000, 1536, 2304, 2, "random"),
    (2600, 1280, 4352, 1, "equal"),
    # a single row tile left over after the blocks of 4 joins the last block: 9 row tiles x 10 column panels in
    # forward (4 + 5), 5 x 10 in the weight gradient (one block of 5), and a ragged pair of groups with 5 row tiles each
    (2300, 1280, 2560, 1, "equal"),
    (2100, 768, 1024, 2, "equal"),
    # many groups of a few row tiles each: whole groups go to single XCDs (lists per XCD) in forward and dX
    (32768, 256, 1280, 64, "equal"),
    (20000, 320, 768, 24, "equal"),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N,E,kind", GMM_CASES)
def test_forward_and_backward_vs_oracle(M, K, N, E, kind, dtype, device):
    say("gmm case", M, K, N, E, kind, dtype)
    gen = torch.Generator().manual_seed(M + K + N)
    counts = _counts(kind, E, M, seed=M)
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, N, generator=gen) * 0.05).to(dtype)
    gy = torch.randn(M, N, generator=gen).to(dtype)
    exp_y = O.gmm(x, w, counts, 0, 1)
    exp_dx, exp_dw = O.gmm_backward(gy, x, w, counts, 1)

    xd = x.to(device).requires_grad_(True)
    wd = w.to(device).requires_grad_(True)
    y = ops.npu_gmm_v2(xd, wd, group_list=counts.to(device), group_type=0)
    y.backward(gy.to(device))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert y.shape == (M, N) and rel_l2(y, exp_y) <= tol
    assert rel_l2(xd.grad, exp_dx) <= tol
    assert wd.grad.shape == w.shape and rel_l2(wd.grad, exp_dw) <= tol
    for gidx in torch.nonzero(counts == 0).flatten().tolist():
        assert torch.count_nonzero(wd.grad[gidx]) == 0          # empty group => zero dW block
    # fp64 bound
    y64 = O.gmm(x.double(), w.double(), counts, 0, 1)
    assert rel_l2(y, y64) <= tol
    # cumulative list form gives the same bits
    y2 = ops.npu_gmm(x.to(device), w.to(device), group_list=torch.cumsum(counts, 0).tolist(), group_type=0)
    assert torch.equal(y2, y.detach())


@pytest.mark.parametrize("E,empty,K,N,rows", [
    (17, (16,), 2048, 4096, 256),          # 16 groups of 256 rows and one empty: the XCD with three groups has 3 x 128 tiles
    (20, (3, 8, 13, 19), 2880, 2880, 192),  # 16 + 4 empty, 12 x 12 output tiles per group
    (23, (), 1024, 2048, 128),             # no empty group; 23 groups deal out as 3, 3, 3, 3, 3, 3, 3, 2
])
def test_weight_gradient_group_count_not_a_multiple_of_8(E, empty, K, N, rows, device):
    """Split on the reduction dim with whole groups dealt out to single XCDs: the XCD with the most groups holds
    ceil(E / 8) whole output blocks, more than an eighth of all tiles when E is not a multiple of 8 (with empty groups
    ranked last the reduction lengths still balance, so the lists are taken).  Every tile of every block must be
    written, and an empty group's block must be exactly zero (test_npu_gmm.py:105-113 in the reference).  The output
    buffer is poisoned first through the caching allocator."""
    say("dW lists", E, empty, K, N, rows)
    counts = torch.tensor([0 if g in empty else rows for g in range(E)])
    M = int(counts.sum())
    gen = torch.Generator().manual_seed(E)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    gy = torch.randn(M, N, generator=gen).to(torch.bfloat16)
    exp = O.gmm(x.t(), gy, counts, 2, 1)
    xd, gyd, gl = x.to(device), gy.to(device), counts.to(device)
    for form in ("counts", "cumulative"):
        poison = torch.full((E, K, N), float("nan"), dtype=torch.bfloat16, device=device)
        del poison
        if form == "counts":
            got = ops.npu_gmm_v2(xd.t(), gyd, group_list=gl, group_type=2)
        else:
            got = ops.npu_gmm(xd.t(), gyd, group_list=torch.cumsum(counts, 0).tolist(), group_type=2)
        torch.cuda.synchronize()
        assert got.shape == (E, K, N)
        assert not torch.isnan(got).any(), "tiles of the weight gradient were left unwritten"
        assert rel_l2(got, exp) <= 1e-2
        for g in empty:
            assert torch.count_nonzero(got[g]) == 0
    # the fp32 `+=` form (npu_groupmatmul_add_fp32) on the same launch shape
    acc = torch.ones(E * K, N, dtype=torch.float32, device=device)
    ops.npu_groupmatmul_add_fp32(xd, gyd, torch.cumsum(counts, 0).to(device), acc)
    torch.cuda.synchronize()
    assert rel_l2(acc.view(E, K, N) - 1.0, exp.float()) <= 1e-2
    for g in empty:
        assert torch.equal(acc.view(E, K, N)[g], torch.ones(K, N, device=device))


def test_transposed_weight_view_and_raw_module(device):
    """A weight stored [E, N, K] and passed as .transpose(1, 2) (Ops.gmm's trans_b form) needs no copy."""
    gen = torch.Generator().manual_seed(5)
    M, K, N, E = 700, 192, 320, 4
    counts = _counts("random", E, M, 5)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    wt = (torch.randn(E, N, K, generator=gen) * 0.05).to(torch.bfloat16)
    exp = O.gmm(x, wt.transpose(1, 2), counts, 0, 1)
    got = ops.npu_gmm_v2(x.to(device), wt.to(device).transpose(1, 2), group_list=counts.to(device))
    assert rel_l2(got, exp) <= 1e-2
    # raw list-in / list-out module used by BaseGMMFunction subclasses
    mod = ops.GMMFunction.builder.load()
    cum = torch.cumsum(counts, 0).to(device)
    w = wt.transpose(1, 2).contiguous().to(device)
    (y,) = mod.npu_gmm([x.to(device)], [w], [], cum, 0, 0)
    gy = torch.randn(M, N, generator=gen).to(torch.bfloat16)
    dx, dw, dbias = mod.npu_gmm_backward([gy.to(device)], [x.to(device)], [w], cum, 0)
    e_dx, e_dw = O.gmm_backward(gy, x, w.cpu(), counts, 1)
    assert rel_l2(y, exp) <= 1e-2 and rel_l2(dx[0], e_dx) <= 1e-2 and rel_l2(dw[0], e_dw) <= 1e-2 and dbias == []
    dx2, dw2, _ = mod.npu_gmm_backward_fusion([gy.to(device)], [w], cum, 0)
    assert torch.equal(dx2[0], dx[0]) and dw2 == []


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_row_contiguous_x_with_split_on_rows(dtype, device):
    """x handed over as the transposed view of a [K, M] buffer (unit stride along its rows) with a split on rows:
    groups of 3, 13 and 0 rows start and end off the 8-row chunks such an operand is fetched in."""
    gen = torch.Generator().manual_seed(11)
    counts = torch.tensor([3, 13, 0, 40, 8, 64])
    M, K, N = int(counts.sum()), 64, 96
    xt = torch.randn(K, M, generator=gen).to(dtype)
    w = (torch.randn(len(counts), K, N, generator=gen) * 0.05).to(dtype)
    exp = O.gmm(xt.t().contiguous(), w, counts, 0, 1)
    x_view = xt.to(device).t()
    assert x_view.stride(0) == 1
    got = ops.npu_gmm_v2(x_view, w.to(device), group_list=counts.to(device), group_type=0)
    assert rel_l2(got, exp) <= TOL[dtype]
    got = ops.npu_gmm(x_view, w.to(device), group_list=torch.cumsum(counts, 0).tolist(), group_type=0)
    assert rel_l2(got, exp) <= TOL[dtype]
    # the same view with a transposed weight view (both operands off their usual layouts)
    wt = w.transpose(1, 2).contiguous().to(device).transpose(1, 2)
    got = ops.npu_gmm_v2(x_view, wt, group_list=counts.to(device), group_type=0)
    assert rel_l2(got, exp) <= TOL[dtype]


def test_rows_past_last_offset_are_zero(device):
    gen = torch.Generator().manual_seed(6)
    x = torch.randn(600, 64, generator=gen).to(torch.bfloat16).to(device)
    w = torch.randn(3, 64, 96, generator=gen).to(torch.bfloat16).to(device)
    y = ops.npu_gmm(x, w, group_list=[100, 100, 430], group_type=0)
    exp = O.gmm(x.cpu(), w.cpu(), [100, 100, 430], 0, 0)
    assert torch.count_nonzero(y[430:]) == 0 and rel_l2(y, exp) <= 1e-2


def test_gemm_fusion_accumulates_into_main_grad(device):
    """gemm_fusion=True: dW is added into original_weight.main_grad (fp32) and a dummy grad is returned
    (mindspeed/ops/gmm.py:56-89)."""
    gen = torch.Generator().manual_seed(8)
    M, K, N, E = 512, 96, 160, 4
    counts = _counts("skew_empty", E, M, 8)
    cum = torch.cumsum(counts, 0)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(E, K, N, generator=gen) * 0.05).to(torch.bfloat16)
    gy = torch.randn(M, N, generator=gen).to(torch.bfloat16)
    main0 = torch.randn(E * K, N, generator=gen)
    param = torch.nn.Parameter(w.to(device))
    param.main_grad = main0.clone().to(device)
    param.grad_added_to_main_grad = False
    xd = x.to(device).requires_grad_(True)
    y = ops.npu_gmm(xd, param, group_list=cum.to(device), group_type=0, gemm_fusion=True, original_weight=param)
    y.backward(gy.to(device))
    exp_dx, _ = O.gmm_backward(gy, x, w, counts, 1)
    exp_main = O.groupmatmul_add_fp32(x, gy, cum, main0.clone())
    assert param.grad_added_to_main_grad is True
    assert rel_l2(xd.grad, exp_dx) <= 1e-2
    assert rel_l2(param.main_grad, exp_main) <= 1e-5
    # v2 (counts) form
    param.main_grad = main0.clone().to(device)
    xd2 = x.to(device).requires_grad_(True)
    ops.npu_gmm_v2(xd2, param, group_list=counts.to(device), gemm_fusion=True, original_weight=param).backward(gy.to(device))
    assert rel_l2(param.main_grad, exp_main) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K,N", [(600, 520), (256, 256), (1032, 392)])
def test_groupmatmul_add_reduction_lengths(K, N, dtype, device):
    """The fp32 `+=` form over groups of 0 to 1000 rows (none, one, three, four, five and many K steps: its first old
    values are requested from inside the K loop only where a group has at least four), output blocks whose last row and
    column tiles are partly filled, twice in a row into the same buffer."""
    say("groupmatmul_add reduction lengths", K, N, dtype)
    counts = [0, 1, 31, 32, 96, 127, 128, 129, 1000, 0, 160, 333]
    M = sum(counts)
    gen = torch.Generator().manual_seed(K + N)
    x = torch.randn(M, K, generator=gen).to(dtype)
    dy = torch.randn(M, N, generator=gen).to(dtype)
    acc0 = torch.randn(len(counts) * K, N, generator=gen)
    offsets = torch.cumsum(torch.tensor(counts), 0)
    acc = acc0.clone().to(device)
    xd, dyd, od = x.to(device), dy.to(device), offsets.to(device)
    ops.npu_groupmatmul_add_fp32(xd, dyd, od, acc)
    exp = O.groupmatmul_add_fp32(x, dy, offsets, acc0.clone())
    assert rel_l2(acc, exp) <= 1e-5
    empty = [g for g, c in enumerate(counts) if c == 0]
    for g in empty:                                  # nothing added: the old values exactly
        assert torch.equal(acc[g * K:(g + 1) * K].cpu(), acc0[g * K:(g + 1) * K])
    ops.npu_groupmatmul_add_fp32(xd, dyd, od, acc)
    exp2 = O.groupmatmul_add_fp32(x, dy, offsets, exp.clone())
    assert rel_l2(acc, exp2) <= 1e-5


def test_groupmatmul_add_many_groups(device):
    """The fp32 `+=` form with 24 near-equal groups (whole output blocks dealt out to single XCDs)."""
    say("groupmatmul_add many groups")
    counts = [200 + 9 * (i % 7) for i in range(24)]
    M, K, N = sum(counts), 512, 520
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    dy = torch.randn(M, N, generator=gen).to(torch.bfloat16)
    acc0 = torch.randn(len(counts) * K, N, generator=gen)
    offsets = torch.cumsum(torch.tensor(counts), 0)
    acc = acc0.clone().to(device)
    ops.npu_groupmatmul_add_fp32(x.to(device), dy.to(device), offsets.to(device), acc)
    assert rel_l2(acc, O.groupmatmul_add_fp32(x, dy, offsets, acc0.clone())) <= 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
def test_forward_bias(dtype, device):
    """``bias [E, N]`` is added to every row of its group in the forward pass (docs/zh/ops/gmm.md: forward only; a
    bias that requires a gradient is refused, mindspeed/ops/gmm.py:27-28); rows past the last offset stay zero, and
    the gradients of x and weight are what they are without it."""
    say("forward bias", dtype)
    gen = torch.Generator().manual_seed(17)
    counts = [130, 0, 300, 77, 1, 64]
    M, K, N, E, extra = sum(counts), 96, 160, len(counts), 9
    x = torch.randn(M + extra, K, generator=gen).to(dtype)
    w = (torch.randn(E, K, N, generator=gen) * 0.1).to(dtype)
    bias = torch.randn(E, N, generator=gen).to(torch.float32 if dtype == torch.bfloat16 else dtype)
    cum = torch.cumsum(torch.tensor(counts), 0)
    exp = torch.zeros(M + extra, N, dtype=torch.float64)
    exp[:M] = O.grouped_matmul(x[:M].double(), counts, w.double()) + torch.repeat_interleave(bias.double(), torch.tensor(counts), dim=0)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    for y in (ops.npu_gmm(xd, wd, bias=bias.to(device), group_list=cum.tolist(), group_type=0),
              ops.npu_gmm(xd, wd, bias=bias.to(device), group_list=cum.to(device), group_type=0),
              ops.npu_gmm_v2(xd, wd, bias=bias.to(device), group_list=torch.tensor(counts, device=device), group_type=0)):
        assert y.dtype == dtype and rel_l2(y, exp) <= TOL[dtype]
        assert torch.count_nonzero(y[M:]) == 0
    gy = torch.randn(M + extra, N, generator=gen).to(dtype)
    y.backward(gy.to(device))
    e_dx, e_dw = O.gmm_backward(gy[:M], x[:M], w, counts, 1)
    assert rel_l2(xd.grad[:M], e_dx) <= TOL[dtype] and rel_l2(wd.grad, e_dw) <= TOL[dtype]
    with pytest.raises(ValueError, match="gradient"):
        ops.npu_gmm(xd, wd, bias=bias.to(device).requires_grad_(True), group_list=cum.tolist(), group_type=0)
    with pytest.raises(ValueError, match="bias"):
        ops.npu_gmm(xd.detach().t()[:, :M], torch.randn(M, N).to(dtype).to(device), bias=bias.to(device),
                    group_list=cum.tolist(), group_type=2)
    with pytest.raises(ValueError, match="bias must be"):
        ops.npu_gmm(xd, wd, bias=bias[:, :8].to(device), group_list=cum.tolist(), group_type=0)


def test_linearity_at_mixtral_fc1_shape(device):
    """Full-size property check on the Mixtral fc1 shape: gmm(a*x1 + x2) == a*gmm(x1) + gmm(x2) within bf16
    rounding, and sampled rows against per-row fp32 matmuls."""
    T, H, F, E = 8192, 4096, 14336, 8
    say("mixtral fc1 linearity")
    gen = torch.Generator(device=device).manual_seed(0)
    w = (torch.randn(E, H, 2 * F, generator=gen, device=device) * 0.02).to(torch.bfloat16)
    x1 = torch.randn(T, H, generator=gen, device=device).to(torch.bfloat16)
    counts = torch.tensor([1100, 900, 1024, 1024, 1200, 848, 1000, 1096], device=device)
    y1 = ops.npu_gmm_v2(x1, w, group_list=counts)
    y2 = ops.npu_gmm_v2(x1 * 2, w, group_list=counts)                 # exact scaling in bf16
    assert torch.equal(y2, y1 * 2)
    rows = torch.randint(0, T, (48,), generator=torch.Generator().manual_seed(1))
    bounds = torch.cumsum(counts.cpu(), 0)
    for r in rows.tolist():
        g = int(torch.searchsorted(bounds, torch.tensor(r), right=True))
        ref = x1[r].float().cpu() @ w[g].float().cpu()
        assert rel_l2(y1[r], ref) <= 1e-2, r


# Launches that end in a round of small tail tiles over a long reduction: 31 or 32 row tiles of 256 rows in front
# (8 column panels: 248 / 256 tiles on 256 compute units), then the 64- / 128-row tails, whose reduction the larger
# workspace lets the library cut into parts.
SPLIT_CASES = [
    # counts (sum 8192 + ...), k, n
    ([2098, 2049, 2148, 1897], 4096, 2048),          # two parts per tail
    ([2098, 2049, 2148, 1897], 8264, 2048),          # four parts, the last one shorter and not a multiple of 64
    ([2048, 2049, 2048, 2048 + 120], 16384, 2048),   # complete last round of full tiles; 1- and 120-row tails
]


def _gmm_abi(x, w, counts_dev, n, split, out):
    """ms_gmm through ctypes with the plain or the larger (tail-splitting) workspace."""
    import ctypes
    from mindspeed_amd import _lib
    lib = _lib.load()
    m, k = x.shape
    E = counts_dev.numel()
    dt = _lib.dtype_code(x.dtype, "x")
    nb = ctypes.c_size_t(0)
    if split:
        _lib.check(lib.ms_gmm_workspace_size_split(E, m, k, n, 0, dt, dt, 0, ctypes.byref(nb)), "size")
    else:
        _lib.check(lib.ms_gmm_workspace_size(E, m, 0, ctypes.byref(nb)), "size")
    ws = torch.empty(nb.value, dtype=torch.uint8, device=x.device)
    _lib.check(lib.ms_gmm(_lib.stream_ptr(x.device), _lib.ptr(x), x.stride(0), x.stride(1), _lib.ptr(w), w.stride(0),
                          w.stride(1), w.stride(2), _lib.ptr(out), n, _lib.ptr(counts_dev), 1, 0, E, m, k, n, dt, dt, 0,
                          _lib.ptr(ws), ws.numel()), "ms_gmm")
    torch.cuda.synchronize()
    return nb.value


@pytest.mark.parametrize("counts,K,N,transposed,dtype",
                         [(c, k, n, t, torch.bfloat16) for c, k, n in SPLIT_CASES for t in (False, True)] +
                         [(*SPLIT_CASES[0], False, torch.float16), (*SPLIT_CASES[0], True, torch.float16)])
def test_split_tail_tiles(counts, K, N, transposed, dtype, device):
    """Tail tiles computed in parts along the reduction: rows outside the tails are bit-equal to the unsplit launch,
    the tail rows match the oracle (fp32 CPU evaluation of just those rows) as closely as the unsplit launch does,
    and the Python surface (which asks for the larger workspace) returns the split result."""
    say("split tails", counts, K, N, transposed, dtype)
    gen = torch.Generator().manual_seed(7)
    M, E = sum(counts), len(counts)
    x = torch.randn(M, K, generator=gen).to(dtype).to(device)
    if transposed:
        w = (torch.randn(E, N, K, generator=gen) * 0.05).to(dtype).to(device).transpose(1, 2)
    else:
        w = (torch.randn(E, K, N, generator=gen) * 0.05).to(dtype).to(device)
    cdev = torch.tensor(counts, dtype=torch.int64, device=device)
    plain = torch.full((M, N), float("nan"), dtype=dtype, device=device)
    split = torch.full((M, N), float("nan"), dtype=dtype, device=device)
    small = _gmm_abi(x, w, cdev, N, False, plain)
    large = _gmm_abi(x, w, cdev, N, True, split)
    assert large > small + (1 << 20)
    ends = np.cumsum(counts)
    tail_rows = []
    for c, end in zip(counts, ends):
        rem = c - (c - 1) // 256 * 256
        if rem <= 128:
            tail_rows += list(range(end - rem, end))
    tail = torch.zeros(M, dtype=torch.bool)
    tail[tail_rows] = True
    assert torch.equal(plain[~tail.to(device)], split[~tail.to(device)])
    assert not torch.isnan(split.float()).any()
    # a different summation order over thousands of values leaves rounding differences somewhere in the tail rows:
    # the larger workspace did take the split path
    assert not torch.equal(plain[tail.to(device)], split[tail.to(device)])
    # oracle on the tail rows only, group by group
    xc, wc = x.cpu(), w.cpu()
    start = 0
    for g, (c, end) in enumerate(zip(counts, ends)):
        rows = [r for r in tail_rows if start <= r < end]
        if rows:
            want = O.grouped_matmul(xc[rows], [len(rows)], wc[g:g + 1]).float()
            e_split, e_plain = rel_l2(split[rows].float().cpu(), want), rel_l2(plain[rows].float().cpu(), want)
            say("  group", g, "rows", len(rows), "rel-L2 split / plain", e_split, e_plain)
            assert e_split <= TOL[dtype] and e_split <= 1.5 * e_plain + 1e-4
        start = end
    got = ops.npu_gmm_v2(x, w, group_list=cdev, group_type=0)
    assert torch.equal(got, split)


def test_split_tail_tiles_with_rows_past_the_last_offset(device):
    """The tail split next to the zero-fill of rows that no group covers: those rows are zeros in both launches, the
    rest matches as in test_split_tail_tiles."""
    say("split tails + rows past the last offset")
    counts, K, N, extra = [2098, 2049, 2148, 1897], 4096, 2048, 300
    gen = torch.Generator().manual_seed(9)
    M = sum(counts) + extra
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16).to(device)
    w = (torch.randn(len(counts), K, N, generator=gen) * 0.05).to(torch.bfloat16).to(device)
    cdev = torch.tensor(counts, dtype=torch.int64, device=device)
    plain = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=device)
    split = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=device)
    _gmm_abi(x, w, cdev, N, False, plain)
    _gmm_abi(x, w, cdev, N, True, split)
    covered = sum(counts)
    assert torch.equal(split[covered:], torch.zeros(extra, N, dtype=torch.bfloat16, device=device))
    assert torch.equal(plain[covered:], split[covered:])
    assert not torch.isnan(split.float()).any()
    assert rel_l2(split[:covered].float().cpu(), plain[:covered].float().cpu()) <= 2e-3
    full = torch.ones(M, dtype=torch.bool)
    for c, end in zip(counts, np.cumsum(counts)):
        rem = c - (c - 1) // 256 * 256
        if rem <= 128:
            full[end - rem:end] = False
    full[covered:] = False
    assert torch.equal(plain[full.to(device)], split[full.to(device)])


def test_many_small_groups_take_whole_groups_per_xcd(device):
    """Near-equal ragged groups of two to five row tiles, 40 of them, and rows past the last offset: the launch deals
    whole groups out to single XCDs; forward, dX and dW against the oracle, the uncovered rows zero."""
    say("many small groups")
    gen = torch.Generator().manual_seed(21)
    E, K, N, extra = 40, 384, 1536, 300
    counts = torch.randint(600, 1200, (E,), generator=gen)
    M = int(counts.sum())
    x = torch.randn(M + extra, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(E, K, N, generator=gen) * 0.05).to(torch.bfloat16)
    gy = torch.randn(M + extra, N, generator=gen).to(torch.bfloat16)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    y = ops.npu_gmm_v2(xd, wd, group_list=counts.to(device), group_type=0)
    y.backward(gy.to(device))
    ey = O.grouped_matmul(x[:M], counts.tolist(), w)
    assert rel_l2(y[:M], ey) <= TOL[torch.bfloat16]
    assert torch.equal(y[M:].cpu(), torch.zeros(extra, N, dtype=torch.bfloat16))
    edx, edw = O.gmm_backward(gy[:M], x[:M], w, torch.cumsum(counts, 0).tolist())
    assert rel_l2(xd.grad[:M], edx) <= TOL[torch.bfloat16] and rel_l2(wd.grad, edw) <= TOL[torch.bfloat16]
    assert torch.equal(xd.grad[M:].cpu(), torch.zeros(extra, K, dtype=torch.bfloat16))
