"""Pins the CPU oracle (oracle/) with checks that do not restate its formulas:
brute force on tiny inputs, library routines, invariants, autograd, and the
committed golden fixtures.  Runs without a GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from oracle import permute_index as PI

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _golden(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


# ---- permute ------------------------------------------------------------------------
def test_worked_example_fixture():
    g = _golden("worked_example.npz")
    tokens = torch.from_numpy(g["tokens"])
    indices = torch.from_numpy(g["indices"])
    permuted, sorted_indices = O.permute(tokens, indices)
    assert sorted_indices.tolist() == g["sorted_indices"].tolist()
    assert torch.equal(permuted, torch.from_numpy(g["permuted"]))
    assert O.row_id_map(indices).tolist() == g["row_id_map"].tolist()
    out = O.unpermute(permuted, sorted_indices, torch.from_numpy(g["probs"]))
    assert torch.equal(out, torch.from_numpy(g["unpermuted"]))
    out2 = O.fused_unpermute(permuted, O.row_id_map(indices), torch.from_numpy(g["probs"]))
    assert torch.equal(out2, torch.from_numpy(g["unpermuted"]))


@pytest.mark.parametrize("T,k,E,seed", [(1, 1, 1, 0), (7, 2, 3, 1), (33, 4, 5, 2), (64, 8, 64, 3), (200, 2, 8, 4)])
def test_permute_order_bruteforce_numpy_and_c(T, k, E, seed):
    gen = torch.Generator().manual_seed(seed)
    indices = torch.randint(0, E, (T, k), generator=gen)
    flat = indices.reshape(-1).tolist()
    brute = sorted(range(len(flat)), key=lambda i: (flat[i], i))
    _, si = O.permute(torch.zeros(T, 2), indices)
    assert si.tolist() == brute
    assert np.argsort(np.array(flat), kind="stable").tolist() == brute
    fwd, inv, counts = PI.permute_index(np.array(flat), E)
    assert fwd.tolist() == brute
    rm = O.row_id_map(indices)
    assert rm.dtype == torch.int32 and rm.tolist() == inv.tolist()
    # invariants: permutation, monotone keys, ties ascending, inverse relation, histogram
    assert sorted(si.tolist()) == list(range(T * k))
    keys = [flat[i] for i in si.tolist()]
    assert keys == sorted(keys)
    for a, b in zip(range(len(keys) - 1), range(1, len(keys))):
        if keys[a] == keys[b]:
            assert si[a] < si[b]
    assert all(rm[si[r]] == r for r in range(T * k))
    assert counts.tolist() == np.bincount(np.array(flat), minlength=E).tolist()


def test_permute_rows_are_bit_copies_and_drop():
    gen = torch.Generator().manual_seed(5)
    T, k, H = 19, 3, 8
    tokens = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    indices = torch.randint(0, 4, (T, k), generator=gen)
    permuted, si = O.permute(tokens, indices, num_out_tokens=30)
    assert permuted.shape == (30, H) and si.numel() == 30
    for r in range(30):
        assert torch.equal(permuted[r], tokens[si[r] // k])
    fwd, _, _ = PI.permute_index(indices.reshape(-1).numpy(), 4)
    raw = PI.permute_rows(tokens.view(torch.uint8).numpy().reshape(T, -1), fwd, 30, k)
    assert np.array_equal(raw, permuted.view(torch.uint8).numpy().reshape(30, -1))
    fp, fmap = O.fused_permute(tokens, indices, 30)
    assert torch.equal(fp, permuted) and fmap.numel() == T * k
    # negative / zero num_out_tokens rule of the fused op
    assert O.fused_permute(tokens, indices, 0)[0].shape[0] == T * k
    assert O.fused_permute(tokens, indices, -7)[0].shape[0] == T * k - 7
    assert O.fused_permute(tokens, indices, 10 ** 6)[0].shape[0] == T * k


# ---- unpermute -----------------------------------------------------------------------
def test_unpermute_bruteforce_fp64():
    gen = torch.Generator().manual_seed(11)
    T, k, H, E = 23, 4, 6, 5
    x = torch.randn(T * k, H, generator=gen, dtype=torch.float64)
    indices = torch.randint(0, E, (T, k), generator=gen)
    probs = torch.rand(T, k, generator=gen, dtype=torch.float64)
    _, si = O.permute(torch.zeros(T, 1), indices)
    rm = O.row_id_map(indices)
    expect = torch.zeros(T, H, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            for h in range(H):
                expect[t, h] += probs[t, j] * x[rm[t * k + j], h]
    assert torch.allclose(O.unpermute(x, si, probs), expect, rtol=0, atol=1e-12)
    assert torch.allclose(O.fused_unpermute(x, rm, probs), expect, rtol=0, atol=1e-12)


def test_unpermute_inverts_permute():
    gen = torch.Generator().manual_seed(12)
    T, k, H = 40, 4, 16
    tokens = torch.randn(T, H, generator=gen)
    indices = torch.randint(0, 7, (T, k), generator=gen)
    permuted, si = O.permute(tokens, indices)
    probs = torch.full((T, k), 1.0 / k)
    assert torch.equal(O.unpermute(permuted, si, probs), tokens)      # k power of two: exact
    idx1 = torch.randint(0, 7, (T,), generator=gen)
    p1, s1 = O.permute(tokens, idx1)
    assert torch.equal(O.unpermute(p1, s1), tokens)
    assert torch.equal(O.fused_unpermute(p1, O.row_id_map(idx1)), tokens)


def test_dropped_rows_contribute_zero():
    gen = torch.Generator().manual_seed(13)
    T, k, H = 10, 2, 4
    tokens = torch.randn(T, H, generator=gen)
    indices = torch.randint(0, 3, (T, k), generator=gen)
    n = 13
    permuted, rm = O.fused_permute(tokens, indices, n)
    probs = torch.rand(T, k, generator=gen)
    out = O.fused_unpermute(permuted, rm, probs)
    expect = torch.zeros(T, H)
    for t in range(T):
        for j in range(k):
            r = int(rm[t * k + j])
            if r < n:
                expect[t] += probs[t, j] * permuted[r]
    assert torch.allclose(out, expect, atol=1e-6)


def test_backward_formulas_match_autograd():
    gen = torch.Generator().manual_seed(14)
    T, k, H, E = 12, 3, 5, 4
    indices = torch.randint(0, E, (T, k), generator=gen)
    rm = O.row_id_map(indices)
    permuted = torch.randn(T * k, H, generator=gen, dtype=torch.float64, requires_grad=True)
    probs = torch.rand(T, k, generator=gen, dtype=torch.float64, requires_grad=True)
    gy = torch.randn(T, H, generator=gen, dtype=torch.float64)
    out = O.fused_unpermute(permuted, rm, probs)
    gp, gpr = torch.autograd.grad(out, (permuted, probs), gy)
    mp, mpr = O.unpermute_backward(gy, permuted.detach(), rm, probs.detach())
    assert torch.allclose(mp, gp, atol=1e-12) and torch.allclose(mpr, gpr, atol=1e-12)
    tokens = torch.randn(T, H, generator=gen, dtype=torch.float64, requires_grad=True)
    perm, _ = O.permute(tokens, indices)
    gperm = torch.randn(T * k, H, generator=gen, dtype=torch.float64)
    (gt,) = torch.autograd.grad(perm, tokens, gperm)
    assert torch.allclose(O.permute_backward(gperm, rm, k), gt, atol=1e-12)
    assert torch.autograd.gradcheck(lambda a, b: O.fused_unpermute(a, rm, b), (permuted, probs))


# ---- grouped matmul ------------------------------------------------------------------------
def test_gmm_against_library_routines():
    gen = torch.Generator().manual_seed(21)
    E, rows, K, N = 4, 6, 10, 7
    x = torch.randn(E * rows, K, generator=gen, dtype=torch.float64)
    w = torch.randn(E, K, N, generator=gen, dtype=torch.float64)
    bmm = torch.bmm(x.view(E, rows, K), w).reshape(E * rows, N)
    assert torch.allclose(O.grouped_matmul(x, torch.tensor([rows] * E), w), bmm, atol=1e-12)
    assert torch.allclose(O.gmm(x, w, [rows * (i + 1) for i in range(E)], 0, 0), bmm, atol=1e-12)
    assert torch.allclose(O.gmm(x, w, torch.tensor([rows] * E), 0, 1), bmm, atol=1e-12)
    # transposed weight format of the torch path
    assert torch.allclose(O.grouped_matmul(x, torch.tensor([rows] * E), w.transpose(1, 2).contiguous()), bmm, atol=1e-12)
    # single group == mm
    assert torch.allclose(O.gmm(x, w[:1], [E * rows], 0, 0), x @ w[0], atol=1e-12)
    # rows past the last offset are zero
    y = O.gmm(x, w, [3, 5, 9, 11], 0, 0)
    assert torch.count_nonzero(y[11:]) == 0 and torch.allclose(y[5:9], x[5:9] @ w[2], atol=1e-12)


def test_gmm_reference_test_shapes_exact_integers():
    g = _golden("gmm_cases.npz")
    for name in ("rows_a", "rows_b", "rows_doc"):
        counts = g[f"{name}_counts"].tolist()
        x = torch.from_numpy(g[f"{name}_x"]).float()
        w = torch.from_numpy(g[f"{name}_w"]).float()
        y = torch.from_numpy(g[f"{name}_y"]).float()
        for dt in (torch.float32, torch.bfloat16, torch.float16):
            assert torch.equal(O.gmm_split(x.to(dt), w.to(dt), counts, 0).float(), y), (name, dt)
            assert torch.equal(O.gmm(x.to(dt), w.to(dt), torch.tensor(counts), 0, 1).float(), y)
            assert torch.equal(O.gmm(x.to(dt), w.to(dt), np.cumsum(counts).tolist(), 0, 0).float(), y)
    for name in ("red_a", "red_empty"):
        counts = g[f"{name}_counts"].tolist()
        x = torch.from_numpy(g[f"{name}_x"]).float()
        w = torch.from_numpy(g[f"{name}_w"]).float()
        y = torch.from_numpy(g[f"{name}_y"]).float()
        got = O.gmm(x.t(), w, torch.tensor(counts), 2, 1)
        assert got.shape == y.shape and torch.equal(got, y), name
        assert torch.equal(O.gmm_split(x.t(), w, counts, 2).reshape(y.shape), y)
    empty = g["red_empty_y"]
    assert not empty[1].any() and not empty[2].any()      # empty groups give zero blocks


def test_gmm_backward_matches_autograd():
    gen = torch.Generator().manual_seed(22)
    counts = [3, 0, 5, 2]
    x = torch.randn(10, 6, generator=gen, dtype=torch.float64, requires_grad=True)
    w = torch.randn(4, 6, 5, generator=gen, dtype=torch.float64, requires_grad=True)
    gy = torch.randn(10, 5, generator=gen, dtype=torch.float64)
    y = O.gmm_split(x, w, counts, 0)
    gx, gw = torch.autograd.grad(y, (x, w), gy)
    dx, dw = O.gmm_backward(gy, x.detach(), w.detach(), torch.tensor(counts), 1)
    assert torch.allclose(dx, gx, atol=1e-12) and torch.allclose(dw, gw, atol=1e-12)
    assert torch.count_nonzero(dw[1]) == 0


def test_groupmatmul_add_fixture_and_identity():
    g = _golden("groupmatmul_add.npz")
    x = torch.from_numpy(g["x"]).to(torch.bfloat16)
    dy = torch.from_numpy(g["dy"]).to(torch.bfloat16)
    acc = torch.from_numpy(g["acc"]).float()
    got = O.groupmatmul_add_fp32(x, dy, torch.from_numpy(g["offsets"]), acc.clone())
    assert torch.equal(got, torch.from_numpy(g["expect"]).float())
    # the reference test's identity: out + dw
    w = torch.zeros(2, 40, 24, dtype=torch.bfloat16)
    _, dw = O.gmm_backward(dy, x, w, torch.from_numpy(g["offsets"]), 0)
    assert torch.equal(acc + dw.float().reshape(80, 24), got)


# ---- swiglu, chunk sort, whole layer ----------------------------------------------------------
def test_swiglu_closed_form_and_grad():
    gen = torch.Generator().manual_seed(31)
    x = torch.randn(9, 14, generator=gen, dtype=torch.float64, requires_grad=True)
    p = torch.rand(9, generator=gen, dtype=torch.float64, requires_grad=True)
    g, u = x.detach()[:, :7], x.detach()[:, 7:]
    expect = g / (1 + torch.exp(-g)) * u
    assert torch.allclose(O.swiglu(x.detach()), expect, atol=1e-12)
    assert torch.allclose(O.swiglu(x.detach(), p.detach()), expect * p.detach()[:, None], atol=1e-12)
    gy = torch.randn(9, 7, generator=gen, dtype=torch.float64)
    gx, gp = torch.autograd.grad(O.swiglu(x, p), (x, p), gy)
    mx, mp = O.swiglu_backward(gy, x.detach(), p.detach())
    assert torch.allclose(mx, gx, atol=1e-6) and torch.allclose(mp, gp, atol=1e-6)


def test_sort_chunks_bruteforce():
    x = torch.arange(11 * 3, dtype=torch.float32).reshape(11, 3)
    sizes, order = [2, 0, 4, 5], [2, 0, 3, 1]
    out, pr = O.sort_chunks_by_idxs(x, torch.tensor(sizes), torch.tensor(order), torch.arange(11.0))
    starts = np.concatenate([[0], np.cumsum(sizes)])
    rows = [r for i in order for r in range(starts[i], starts[i] + sizes[i])]
    assert torch.equal(out, x[rows]) and pr.tolist() == [float(r) for r in rows]


def test_layer_against_fp64_fixture():
    g = _golden("layer_fp64.npz")
    x, idx, p = (torch.from_numpy(g[k]) for k in ("x", "idx", "p"))
    w1, w2 = torch.from_numpy(g["w1"]), torch.from_numpy(g["w2"])
    out = O.moe_layer(x, idx, p, w1, w2)
    expect = torch.from_numpy(g["out"])
    err = (out.double() - expect).norm() / expect.norm()
    assert err < 1e-6, err
    out64 = O.moe_layer(x.double(), idx, p.double(), w1.double(), w2.double())
    assert (out64 - expect).norm() / expect.norm() < 1e-12


def test_plumbing_config_runs_and_is_consistent():
    # The CPU-runnable configuration: 512 tokens, hidden 256, 8 experts, top-2, FFN 512, fp32, seed 0.
    torch.manual_seed(0)
    T, H, E, K, F = 512, 256, 8, 2, 512
    x = torch.randn(T, H)
    p, idx = O.route_topk(torch.randn(T, E), K)
    w1 = torch.randn(E, H, 2 * F) * 0.02
    w2 = torch.randn(E, F, H) * 0.02
    out = O.moe_layer(x, idx, p, w1, w2)
    dense = torch.zeros(T, H, dtype=torch.float64)
    for e in range(E):
        h = x.double() @ w1[e].double()
        a = torch.nn.functional.silu(h[:, :F]) * h[:, F:]
        y = a @ w2[e].double()
        for j in range(K):
            sel = idx[:, j] == e
            dense[sel] += p[sel, j].double()[:, None] * y[sel]
    assert (out.double() - dense).norm() / dense.norm() < 1e-5


# ---- routing-map (mask) mode ------------------------------------------------------------
def _random_map(T, E, k, seed):
    gen = torch.Generator().manual_seed(seed)
    scores = torch.rand(T, E, generator=gen)
    idx = scores.topk(k, dim=1).indices
    rmap = torch.zeros(T, E, dtype=torch.bool)
    rmap.scatter_(1, idx, True)
    probs = torch.where(rmap, torch.rand(T, E, generator=gen) + 0.1, torch.zeros(T, E))
    return rmap, probs, idx


@pytest.mark.parametrize("T,E,k,seed", [(1, 1, 1, 0), (9, 4, 2, 1), (40, 8, 3, 2), (17, 5, 5, 3)])
def test_routing_map_permute_bruteforce(T, E, k, seed):
    rmap, probs, _ = _random_map(T, E, k, seed)
    gen = torch.Generator().manual_seed(100 + seed)
    tokens = torch.randn(T, 6, generator=gen)
    permuted, pprobs, sidx = O.permute_routing_map(tokens, rmap, probs)
    # brute force: expert-major, token-ascending
    rows = [(e, t) for e in range(E) for t in range(T) if rmap[t, e]]
    assert sidx.tolist() == [t for _, t in rows]
    assert torch.equal(permuted, torch.stack([tokens[t] for _, t in rows]))
    assert torch.equal(pprobs, torch.tensor([probs[t, e].item() for e, t in rows]))
    # unpermute: out[t] = sum over its experts of probs * row
    out = O.unpermute_routing_map(permuted, sidx, tokens.shape, probs, rmap)
    want = torch.zeros(T, 6, dtype=torch.float64)
    for r, (e, t) in enumerate(rows):
        want[t] += probs[t, e].double() * permuted[r].double()
    assert torch.allclose(out.double(), want, rtol=1e-6, atol=1e-6)
    # without probs: plain sum of the rows of a token = k * token
    out1 = O.unpermute_routing_map(permuted, sidx, tokens.shape)
    assert torch.allclose(out1, tokens * k, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("T,E,k,cap,seed", [(9, 4, 2, 3, 1), (12, 3, 1, 6, 2), (10, 5, 2, 10, 3), (16, 4, 2, 1, 4)])
def test_routing_map_drop_and_pad_bruteforce(T, E, k, cap, seed):
    rmap, probs, _ = _random_map(T, E, k, seed)
    gen = torch.Generator().manual_seed(200 + seed)
    tokens = torch.randn(T, 5, generator=gen)
    permuted, pprobs, sidx = O.permute_routing_map(tokens, rmap, probs, num_out_tokens=E * cap, drop_and_pad=True)
    rows = []
    for e in range(E):
        routed = [t for t in range(T) if rmap[t, e]]
        others = [t for t in range(T) if not rmap[t, e]]
        rows += [(e, t) for t in (routed + others)[:cap]]
    assert sidx.tolist() == [t for _, t in rows]
    assert torch.equal(permuted, torch.stack([tokens[t] for _, t in rows]))
    assert torch.equal(pprobs, torch.tensor([probs[t, e].item() for e, t in rows]))
    out = O.unpermute_routing_map(permuted, sidx, tokens.shape, probs, rmap, drop_and_pad=True)
    want = torch.zeros(T, 5, dtype=torch.float64)
    for r, (e, t) in enumerate(rows):
        want[t] += probs[t, e].double() * permuted[r].double()
    assert torch.allclose(out.double(), want, rtol=1e-6, atol=1e-6)


def test_routing_map_mode_agrees_with_index_mode():
    # A map built from top-k indices: the mask form and the index form select the same multiset of rows per
    # expert; with indices sorted inside every token they are the same permutation.
    T, E, k = 50, 8, 2
    rmap, probs, idx = _random_map(T, E, k, 7)
    idx = idx.sort(dim=1).values
    gen = torch.Generator().manual_seed(8)
    tokens = torch.randn(T, 4, generator=gen)
    p_idx, sorted_flat = O.permute(tokens, idx)
    p_map, _, sidx = O.permute_routing_map(tokens, rmap)
    assert torch.equal(p_idx, p_map)
    assert torch.equal(sorted_flat // k, sidx)
    topk_probs = probs.gather(1, idx)
    out_idx = O.unpermute(p_idx, sorted_flat, topk_probs)
    out_map = O.unpermute_routing_map(p_map, sidx, tokens.shape, probs, rmap)
    assert torch.allclose(out_idx, out_map, rtol=1e-6, atol=1e-6)


def test_row_reference_agrees_with_oracle_autograd():
    """The per-row / per-block fp32 evaluation used by the full-size GPU tests (tests/layer_rowref.py) against
    autograd through the whole-layer oracle on a small fp32 configuration: every token, every weight block."""
    from layer_rowref import RowRef

    cfg = dict(T=96, H=40, E=6, K=3, F=24)
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(cfg["T"], cfg["H"], generator=gen)
    p, idx = O.route_topk(torch.randn(cfg["T"], cfg["E"], generator=gen), cfg["K"])
    idx[idx == 4] = 5                                                    # expert 4 gets no rows
    w1 = torch.randn(cfg["E"], cfg["H"], 2 * cfg["F"], generator=gen) * 0.3
    w2 = torch.randn(cfg["E"], cfg["F"], cfg["H"], generator=gen) * 0.3
    gy = torch.randn(cfg["T"], cfg["H"], generator=gen)
    leaves = [t.clone().requires_grad_(True) for t in (x, p, w1, w2)]
    out = O.moe_layer(leaves[0], idx, leaves[1], leaves[2], leaves[3])
    dx, dp, dw1, dw2 = torch.autograd.grad(out, leaves, gy)

    ref = RowRef(cfg, x, p, idx, w1, w2, gy)
    tokens = list(range(cfg["T"]))
    r_out, r_dx, r_dp = ref.token_refs(tokens)
    assert torch.allclose(r_out, out.detach(), rtol=1e-5, atol=1e-5)
    assert torch.allclose(r_dx, dx, rtol=1e-5, atol=1e-5)
    assert torch.allclose(r_dp, dp, rtol=1e-5, atol=1e-5)
    ks, fs, hs = torch.arange(3, 29), torch.arange(5, 24), torch.arange(0, 40, 3)
    for e in range(cfg["E"]):
        g, u, d2 = ref.dw_blocks(e, ks, fs, hs)
        assert torch.allclose(g, dw1[e][ks][:, fs], rtol=1e-5, atol=1e-5)
        assert torch.allclose(u, dw1[e][ks][:, cfg["F"] + fs], rtol=1e-5, atol=1e-5)
        assert torch.allclose(d2, dw2[e][fs][:, hs], rtol=1e-5, atol=1e-5)
    assert ref.counts[4] == 0 and torch.count_nonzero(dw1[4]) == 0


def test_fused_permute_dtype_rule():
    """Result dtypes of the reference's fused permute hook (mindspeed/core/fusions/fused_moe_permute.py:17-47,58-63),
    typed by hand from the rule: promote both to fp32 iff exactly one is fp32, then cast both to the other one's
    dtype.  Values are those of the plain permutation (a gather moves bits) rounded to the result dtype."""
    f32, b16, h16 = torch.float32, torch.bfloat16, torch.float16
    table = {
        (b16, b16): (b16, b16), (b16, f32): (b16, b16), (f32, b16): (b16, b16), (f32, f32): (f32, f32),
        (h16, f32): (h16, h16), (f32, h16): (h16, h16), (h16, h16): (h16, h16),
        (b16, h16): (b16, h16),      # two different 16-bit types: nothing is promoted, nothing is cast
    }
    gen = torch.Generator().manual_seed(4)
    T, E, H = 12, 5, 6
    rmap = torch.rand(T, E, generator=gen) < 0.4
    base_t = torch.randn(T, H, generator=gen)
    base_p = torch.rand(T, E, generator=gen)
    for (tdt, pdt), (want_t, want_p) in table.items():
        tokens, probs = base_t.to(tdt), base_p.to(pdt)
        perm, pp, sidx = O.fused_permute_routing_map(tokens, rmap, probs)
        assert (perm.dtype, pp.dtype) == (want_t, want_p), (tdt, pdt)
        plain_t, plain_p, plain_idx = O.permute_routing_map(tokens, rmap, probs)
        assert torch.equal(sidx, plain_idx)
        assert torch.equal(perm, plain_t.to(want_t)) and torch.equal(pp, plain_p.to(want_p))
    perm, pp, _ = O.fused_permute_routing_map(base_t.to(b16), rmap, None)
    assert perm.dtype == b16 and pp is None
