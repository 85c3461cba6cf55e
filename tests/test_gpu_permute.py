"""GPU parity: token permute / unpermute and their backwards against the CPU
oracle, through the Python surface that calls the C ABI.  Index outputs and
permuted rows are compared bit-exactly; weighted sums within rel-L2 1e-2 (bf16,
fp16) and 1e-5 (fp32)."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

import mindspeed_amd.ops as ops

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-5}


def say(*a):
    print(*a, flush=True)


def routing(T, k, E, seed, skew=0.0):
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=gen) + skew * torch.randn(E, generator=gen)
    p, idx = O.route_topk(logits, k)
    return p, idx


PERMUTE_CASES = [
    # T, k, E, H, dtype, idx dtype, num_out, hint
    (3, 2, 3, 8, torch.float32, torch.int64, None, None),
    (1, 1, 1, 8, torch.bfloat16, torch.int32, None, 1),
    (512, 2, 8, 256, torch.float32, torch.int64, None, 8),
    (97, 3, 5, 72, torch.bfloat16, torch.int64, 200, 5),
    (64, 8, 64, 130, torch.float16, torch.int32, None, None),      # H*2 not a multiple of 16: element path
    (33, 2, 8, 7, torch.float32, torch.int64, None, 8),            # odd hidden, fp32 element path
    (4096, 2, 8, 512, torch.bfloat16, torch.int64, None, 8),       # single-block sort at its R=8192 shape
    (8192, 2, 8, 64, torch.bfloat16, torch.int64, None, None),     # R=16384: largest single-block sort
    (8192, 8, 64, 64, torch.bfloat16, torch.int64, None, 64),      # R=65536: multi-block sort
    (5000, 7, 100, 16, torch.bfloat16, torch.int32, 30000, None),  # ragged, drop, 1024 bins
    (1, 8, 256, 32, torch.bfloat16, torch.int64, None, 256),
    # one launch with per-bin LDS counters (more than 16 bins, R <= 16384)
    (4096, 2, 8, 1024, torch.bfloat16, torch.int64, None, None),   # 1024 bins, 1024-thread workgroups
    (700, 6, 60, 96, torch.float16, torch.int32, 3000, 60),        # 64 bins, drop, top-6
    (2048, 8, 256, 40, torch.float32, torch.int64, None, 256),     # R=16384, 256 bins, 10 lanes per row
    # histogram launch + scatter/rows launch (R > 16384): table summed per workgroup / by its own scan launch
    (4099, 6, 12, 128, torch.bfloat16, torch.int64, None, 12),     # top-6: workgroups straddle segment boundaries
    (3000, 7, 130, 264, torch.bfloat16, torch.int32, 20000, 130),  # 256 bins x 21 segments, drop
    (9000, 4, 40, 32, torch.float32, torch.int64, None, None),     # 1024 bins x 36 segments: scan launch
    (40000, 2, 8, 16, torch.bfloat16, torch.int64, None, 8),       # short rows: 128 rows per workgroup
]


@pytest.mark.parametrize("T,k,E,H,dtype,idt,num_out,hint", PERMUTE_CASES)
def test_permute_bit_exact(T, k, E, H, dtype, idt, num_out, hint, device):
    say("permute case", T, k, E, H, dtype, idt, num_out, hint)
    gen = torch.Generator().manual_seed(T * 31 + k)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    idx = torch.randint(0, E, (T, k), generator=gen).to(idt)
    if k == 1:
        idx = idx.view(-1)
    exp_perm, exp_map = O.fused_permute(tokens, idx, num_out)
    _, exp_sorted = O.permute(tokens, idx, exp_perm.size(0))
    perm, rmap, srt, counts = ops.moe_token_permute_with_aux(tokens.to(device), idx.to(device), num_out,
                                                              num_experts=hint)
    torch.cuda.synchronize()
    assert rmap.dtype == torch.int32 and torch.equal(rmap.cpu(), exp_map)
    assert torch.equal(srt.cpu().long(), exp_sorted)
    assert perm.shape == exp_perm.shape and torch.equal(perm.cpu().view(torch.uint8), exp_perm.view(torch.uint8))
    if hint is not None:
        assert torch.equal(counts.cpu(), torch.bincount(idx.reshape(-1).long(), minlength=hint))
    # reference-signature entry point returns the same pair
    p2, m2 = ops.npu_moe_token_permute(tokens.to(device), idx.to(device), num_out)
    assert torch.equal(p2, perm) and torch.equal(m2, rmap)


def test_permute_worked_example_fixture(device):
    g = np.load(os.path.join(GOLDEN, "worked_example.npz"))
    perm, rmap, srt, counts = ops.moe_token_permute_with_aux(
        torch.from_numpy(g["tokens"]).to(device), torch.from_numpy(g["indices"]).to(device), num_experts=3)
    assert rmap.cpu().tolist() == g["row_id_map"].tolist()
    assert srt.cpu().tolist() == g["sorted_indices"].tolist()
    assert counts.cpu().tolist() == g["tokens_per_expert"].tolist()
    assert torch.equal(perm.cpu(), torch.from_numpy(g["permuted"]))
    out = ops.npu_moe_token_unpermute(perm, rmap, torch.from_numpy(g["probs"]).to(device))
    assert torch.equal(out.cpu(), torch.from_numpy(g["unpermuted"]))


def test_permute_empty_and_negative_num_out(device):
    tokens = torch.randn(6, 8, device=device).to(torch.bfloat16)
    idx = torch.randint(0, 3, (6, 2), device=device)
    perm, rmap = ops.npu_moe_token_permute(tokens, idx, -4)            # n + T*k rows
    exp_perm, exp_map = O.fused_permute(tokens.cpu(), idx.cpu(), -4)
    assert perm.shape[0] == 8 and torch.equal(perm.cpu(), exp_perm) and torch.equal(rmap.cpu(), exp_map)
    e_perm, e_map = ops.npu_moe_token_permute(tokens[:0], idx[:0])
    assert e_perm.shape == (0, 8) and e_map.numel() == 0


@pytest.mark.parametrize("idt", [torch.int32, torch.int64])
@pytest.mark.parametrize("T,E", [(300, 8), (4096, 8), (1000, 16), (700, 200)])
def test_permute_out_of_range_ids_are_clamped(idt, T, E, device):
    """Expert ids outside [0, num_experts) are clamped into range before sorting (negative ones to the first
    expert, large ones to the last bin), for every index width, also when only the upper half of a 64-bit id is
    set.  The bins are a power of two, so ids up to the next power of two keep their own bin."""
    say("permute clamp case", idt, T, E)
    k, H = 2, 64
    gen = torch.Generator().manual_seed(T + E)
    idx = torch.randint(0, E, (T, k), generator=gen).to(idt)
    nbins = 2
    while nbins < E:
        nbins *= 2
    odd = [-1, -7, nbins, nbins + 100, 2 ** 31 - 1]
    if idt == torch.int64:
        odd += [2 ** 33 + 3, -(2 ** 40), 2 ** 62]
    where = torch.randperm(T * k, generator=gen)[:len(odd) * 3]
    flat = idx.view(-1)
    for i, pos in enumerate(where.tolist()):
        flat[pos] = odd[i % len(odd)]
    clamped = idx.clamp(0, nbins - 1)
    tokens = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    exp_perm, exp_map = O.fused_permute(tokens, clamped, None)
    _, exp_sorted = O.permute(tokens, clamped, exp_perm.size(0))
    perm, rmap, srt, counts = ops.moe_token_permute_with_aux(tokens.to(device), idx.to(device), None, num_experts=E)
    torch.cuda.synchronize()
    assert torch.equal(rmap.cpu(), exp_map)
    assert torch.equal(srt.cpu().long(), exp_sorted)
    assert torch.equal(perm.cpu(), exp_perm)
    assert torch.equal(counts.cpu(), torch.bincount(clamped.reshape(-1).long(), minlength=nbins)[:E])


UNPERMUTE_CASES = [
    (512, 2, 8, 256, torch.float32, None),
    (300, 4, 16, 136, torch.bfloat16, None),
    (128, 8, 64, 2048, torch.bfloat16, None),
    (77, 3, 6, 50, torch.float16, None),        # element path
    (200, 2, 8, 64, torch.bfloat16, 250),       # dropped rows
    (4096, 2, 8, 1024, torch.bfloat16, None),
]


@pytest.mark.parametrize("T,k,E,H,dtype,num_out", UNPERMUTE_CASES)
def test_unpermute_forward_backward(T, k, E, H, dtype, num_out, device):
    say("unpermute case", T, k, E, H, dtype, num_out)
    p, idx = routing(T, k, E, seed=T + k)
    gen = torch.Generator().manual_seed(7)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    probs = p.to(dtype)
    exp_perm, exp_map = O.fused_permute(tokens, idx, num_out)
    rows = exp_perm.size(0)
    x = (torch.randn(rows, H, generator=gen)).to(dtype)
    gy = torch.randn(T, H, generator=gen).to(dtype)
    exp_out = O.fused_unpermute(x, exp_map, probs)
    exp_gx, exp_gp = O.unpermute_backward(gy, x, exp_map, probs)

    xd = x.to(device).requires_grad_(True)
    pd = probs.to(device).requires_grad_(True)
    out = ops.npu_moe_token_unpermute(xd, exp_map.to(device), pd)
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert rel_l2(out, exp_out) <= tol
    assert rel_l2(xd.grad, exp_gx) <= tol
    assert rel_l2(pd.grad, exp_gp) <= tol
    # fp64 brute force (informational bound, same tolerance)
    ref64 = O.fused_unpermute(x.double(), exp_map, probs.double())
    assert rel_l2(out, ref64) <= tol

    # probs=None: topk taken as 1 (npu_moe_token_unpermute.cpp:108), plain inverse gather
    if num_out is None:
        idx1 = idx[:, 0].contiguous()
        perm1, map1 = ops.npu_moe_token_permute(tokens.to(device), idx1.to(device))
        back = ops.npu_moe_token_unpermute(perm1, map1)
        assert torch.equal(back.cpu(), tokens)


@pytest.mark.parametrize("tdtype,pdtype", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                           (torch.float32, torch.bfloat16)])
def test_unpermute_probs_keep_their_own_dtype(tdtype, pdtype, device):
    """Probabilities of another dtype than the tokens are used unrounded (the torch path multiplies bf16 tokens by
    fp32 probabilities in fp32, mindspeed/core/transformer/moe/moe_utils.py:236-238), and their gradient is an fp32
    dot product stored in the probabilities' dtype."""
    say("unpermute mixed dtypes", tdtype, pdtype)
    T, k, E, H = 256, 2, 8, 512
    _, idx = routing(T, k, E, seed=3)
    exp_map = O.fused_permute(torch.zeros(T, 1), idx, None)[1]
    if pdtype == torch.float32:
        # 1024 * (0.5 + 2^-11) - 1024 * 0.5 = 0.5 exactly; with the probabilities rounded to 16 bits first it is 0
        x = torch.empty(T * k, H)
        x[exp_map.long()] = torch.tensor([1024.0, -1024.0]).repeat(T)[:, None].expand(T * k, H)
        probs = torch.tensor([0.5 + 2.0 ** -11, 0.5]).repeat(T, 1)
        out = ops.npu_moe_token_unpermute(x.to(tdtype).to(device), exp_map.to(device), probs.to(device))
        assert out.dtype == tdtype
        assert torch.equal(out.float().cpu(), torch.full((T, H), 0.5))
    gen = torch.Generator().manual_seed(11)
    x = torch.randn(T * k, H, generator=gen).to(tdtype)
    gy = torch.randn(T, H, generator=gen).to(tdtype)
    probs = torch.rand(T, k, generator=gen).to(pdtype)
    xd = x.to(device).requires_grad_(True)
    pd = probs.to(device).requires_grad_(True)
    out = ops.npu_moe_token_unpermute(xd, exp_map.to(device), pd)
    out.backward(gy.to(device))
    torch.cuda.synchronize()
    assert out.dtype == tdtype and pd.grad.dtype == pdtype and xd.grad.dtype == tdtype
    ref = O.fused_unpermute(x.double(), exp_map, probs.double())
    gx, gp = O.unpermute_backward(gy.double(), x.double(), exp_map, probs.double())
    assert rel_l2(out, ref) <= TOL[tdtype]
    assert rel_l2(xd.grad, gx) <= TOL[tdtype]
    # the dot products are exact products of the stored values summed in fp32: fp32 probabilities get them unrounded
    assert rel_l2(pd.grad, gp) <= (1e-5 if pdtype == torch.float32 else TOL[pdtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_permute_backward_and_roundtrip(dtype, device):
    T, k, E, H = 640, 4, 16, 264
    say("permute backward", dtype)
    p, idx = routing(T, k, E, seed=3, skew=1.0)
    gen = torch.Generator().manual_seed(9)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    td = tokens.to(device).requires_grad_(True)
    perm, rmap = ops.npu_moe_token_permute(td, idx.to(device))
    gperm = torch.randn(T * k, H, generator=gen).to(dtype)
    perm.backward(gperm.to(device))
    exp = O.permute_backward(gperm, O.row_id_map(idx), k)
    assert rel_l2(td.grad, exp) <= TOL[dtype]
    # round trip: unpermute(permute(x), 1/k) == x exactly (k power of two)
    probs = torch.full((T, k), 1.0 / k, dtype=dtype, device=device)
    back = ops.npu_moe_token_unpermute(perm.detach(), rmap, probs)
    assert torch.equal(back.cpu(), tokens)


def test_full_size_permute_properties(device):
    """Mixtral-shape (4096 x 4096, top-2, 8 experts) and the 64-expert top-8 shape at full size:
    bit-exact map against the oracle plus size-independent properties."""
    for (T, k, E, H) in ((4096, 2, 8, 4096), (8192, 8, 64, 2048)):
        say("full-size permute", T, k, E, H)
        p, idx = routing(T, k, E, seed=0, skew=1.5 if E == 64 else 0.0)
        gen = torch.Generator().manual_seed(0)
        tokens = torch.randn(T, H, generator=gen).to(torch.bfloat16)
        perm, rmap, srt, counts = ops.moe_token_permute_with_aux(tokens.to(device), idx.to(device), num_experts=E)
        assert torch.equal(rmap.cpu(), O.row_id_map(idx))
        assert torch.equal(counts.cpu(), torch.bincount(idx.reshape(-1), minlength=E))
        s = srt.long()
        assert torch.equal(torch.sort(s)[0], torch.arange(T * k, device=device))          # a permutation
        keys = idx.to(device).reshape(-1)[s]
        assert bool((keys[1:] >= keys[:-1]).all())                                         # sorted by expert
        ties = keys[1:] == keys[:-1]
        assert bool((s[1:][ties] > s[:-1][ties]).all())                                    # stable
        assert torch.equal(rmap.long()[s], torch.arange(T * k, device=device))             # inverse relation
        assert torch.equal(perm, tokens.to(device)[s // k])                                # rows are copies
        probs = torch.full((T, k), 1.0 / k, dtype=torch.bfloat16, device=device)
        assert torch.equal(ops.npu_moe_token_unpermute(perm, rmap, probs).cpu(), tokens)   # round trip
