"""GPU parity: routing-map (mask) mode of permute / unpermute against the CPU oracle, through the Python
surface that calls the C ABI.  Index outputs, permuted rows and permuted probabilities are compared
bit-exactly; weighted sums within rel-L2 1e-2 (bf16, fp16) and 1e-5 (fp32)."""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

from mindspeed_amd.ops import moe_permute_mask_map as M

pytestmark = pytest.mark.gpu
TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float32: 1e-5}


def say(*a):
    print(*a, flush=True)


def make_map(T, E, k, seed, never=()):
    """Top-k style mask and probabilities; experts listed in ``never`` are never chosen."""
    gen = torch.Generator().manual_seed(seed)
    scores = torch.rand(T, E, generator=gen)
    for e in never:
        scores[:, e] = -1.0
    idx = scores.topk(k, dim=1).indices
    rmap = torch.zeros(T, E, dtype=torch.bool)
    rmap.scatter_(1, idx, True)
    probs = torch.where(rmap, torch.rand(T, E, generator=gen) + 0.1, torch.zeros(T, E))
    return rmap, probs


CASES = [
    # T, E, k, H, dtype, probs dtype, never-chosen experts
    (1, 1, 1, 8, torch.bfloat16, torch.float32, ()),
    (9, 4, 2, 16, torch.float32, torch.float32, ()),
    (64, 8, 2, 128, torch.bfloat16, torch.float32, (3,)),
    (300, 8, 2, 264, torch.float32, torch.float32, (0, 7)),
    (257, 5, 3, 70, torch.float16, torch.float16, ()),            # odd hidden: element path
    (512, 64, 8, 96, torch.bfloat16, torch.bfloat16, ()),         # T*E = 32768: multi-block sort
    (4096, 8, 2, 512, torch.bfloat16, torch.float32, ()),         # Mixtral routing at reduced hidden
    (2000, 130, 4, 32, torch.bfloat16, torch.float32, (129,)),    # > 64 experts, ragged
    (200, 8, 2, 64, torch.float32, torch.bfloat16, ()),           # fp32 tokens next to 16-bit probabilities
]


@pytest.mark.parametrize("T,E,k,H,dtype,pdt,never", CASES)
def test_permute_mask_map_forward_backward(T, E, k, H, dtype, pdt, never, device):
    say("routing-map permute case", T, E, k, H, dtype, pdt, never)
    rmap, probs = make_map(T, E, k, T * 7 + E, never)
    probs = probs.to(pdt)
    gen = torch.Generator().manual_seed(T + 13)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    # fused=True: the reference hook's dtype rule (one fp32 operand, one 16-bit one: both results 16-bit);
    # fused=False: Megatron's own permute, every result in its operand's dtype.  Same kernels either way.
    exp_perm, exp_pp, exp_idx = O.fused_permute_routing_map(tokens, rmap, probs)
    plain_perm, plain_pp, _ = O.permute_routing_map(tokens, rmap, probs)

    tok_d = tokens.to(device).requires_grad_(True)
    probs_d = probs.to(device).requires_grad_(True)
    perm_plain, pp_plain, sidx_plain = M.permute(tok_d, rmap.to(device), probs_d, fused=False)
    assert perm_plain.dtype == dtype and pp_plain.dtype == pdt and torch.equal(sidx_plain.cpu(), exp_idx)
    assert torch.equal(perm_plain.detach().cpu(), plain_perm) and torch.equal(pp_plain.detach().cpu(), plain_pp)
    for num_out in (None, exp_perm.size(0)):
        perm, pp, sidx = M.permute(tok_d, rmap.to(device), probs_d, num_out_tokens=num_out, fused=True)
        torch.cuda.synchronize()
        assert sidx.dtype == torch.int64 and torch.equal(sidx.cpu(), exp_idx)
        assert perm.dtype == exp_perm.dtype and torch.equal(perm.detach().cpu(), exp_perm)
        assert pp.dtype == exp_pp.dtype and torch.equal(pp.detach().cpu(), exp_pp)

    # backward: random cotangents for both differentiable outputs
    g_rows = torch.randn(exp_perm.shape, generator=gen).to(exp_perm.dtype)
    g_pp = torch.randn(exp_pp.shape, generator=gen).to(exp_pp.dtype)
    (perm * g_rows.to(device)).sum().backward(retain_graph=True)
    act_grad = tok_d.grad.clone()
    tok_d.grad = None
    (pp * g_pp.to(device)).sum().backward()
    torch.cuda.synchronize()
    t64 = tokens.double().requires_grad_(True)
    p64 = probs.double().requires_grad_(True)
    o_perm, o_pp, _ = O.permute_routing_map(t64, rmap, p64)
    (o_perm * g_rows.double()).sum().backward(retain_graph=True)
    (o_pp * g_pp.double()).sum().backward()
    assert rel_l2(act_grad, t64.grad) <= TOL[dtype]
    assert torch.equal(probs_d.grad.cpu().double(), p64.grad.to(pdt).double())   # a pure scatter of g_pp


@pytest.mark.parametrize("T,E,k,H,dtype,pdt,never", CASES)
@pytest.mark.parametrize("with_probs", [True, False])
def test_unpermute_mask_map_forward_backward(T, E, k, H, dtype, pdt, never, with_probs, device):
    say("routing-map unpermute case", T, E, k, H, dtype, pdt, never, with_probs)
    rmap, probs = make_map(T, E, k, T * 5 + E + 1, never)
    probs = probs.to(pdt)
    gen = torch.Generator().manual_seed(T + 29)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    _, _, sidx = O.permute_routing_map(tokens, rmap)
    rows = torch.randn(sidx.numel(), H, generator=gen).to(dtype)
    g_out = torch.randn(T, H, generator=gen).to(dtype)

    rows_d = rows.to(device).requires_grad_(True)
    probs_d = probs.to(device).requires_grad_(True) if with_probs else None
    out = M.unpermute(rows_d, sidx.to(device), tokens.shape, probs=probs_d, routing_map=rmap.to(device), fused=True)
    out.backward(g_out.to(device))
    torch.cuda.synchronize()

    r64 = rows.double().requires_grad_(True)
    p64 = probs.double().requires_grad_(True) if with_probs else None
    exp = O.unpermute_routing_map(r64, sidx, tokens.shape, p64, rmap)
    exp.backward(g_out.double())
    assert out.dtype == dtype
    assert rel_l2(out, exp) <= TOL[dtype]
    assert rel_l2(rows_d.grad, r64.grad) <= TOL[dtype]
    if with_probs:
        mask = rmap.double()
        # the probabilities' gradient is rounded to their own dtype
        assert rel_l2(probs_d.grad.cpu().double() * mask, p64.grad * mask) <= max(TOL[dtype], TOL[pdt])
        assert torch.count_nonzero(probs_d.grad.cpu().double() * (1 - mask)) == 0   # unset entries get no gradient


PAD_CASES = [
    # T, E, k, capacity, H, dtype
    (9, 4, 2, 3, 16, torch.float32),
    (64, 8, 2, 10, 128, torch.bfloat16),     # some experts over capacity (drop), some under (pad)
    (100, 5, 1, 100, 40, torch.float32),     # capacity = T: every token appears for every expert
    (3000, 8, 2, 700, 64, torch.bfloat16),   # T*E = 24000: multi-block sort, 16 keys
    (500, 16, 4, 1, 8, torch.float16),
]


@pytest.mark.parametrize("T,E,k,cap,H,dtype", PAD_CASES)
def test_drop_and_pad(T, E, k, cap, H, dtype, device):
    say("routing-map drop_and_pad case", T, E, k, cap, H, dtype)
    rmap, probs = make_map(T, E, k, T * 3 + cap)
    gen = torch.Generator().manual_seed(T + 41)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    n = E * cap
    exp_perm, exp_pp, exp_idx = O.fused_permute_routing_map(tokens, rmap, probs, num_out_tokens=n, drop_and_pad=True)
    tok_d = tokens.to(device).requires_grad_(True)
    probs_d = probs.to(device).requires_grad_(True)
    perm, pp, sidx = M.permute(tok_d, rmap.to(device), probs_d, num_out_tokens=n, fused=True, drop_and_pad=True)
    torch.cuda.synchronize()
    assert torch.equal(sidx.cpu(), exp_idx)
    assert torch.equal(perm.detach().cpu(), exp_perm)
    assert pp.dtype == exp_pp.dtype and torch.equal(pp.detach().cpu(), exp_pp)

    g_rows = torch.randn(exp_perm.shape, generator=gen).to(dtype)
    (perm * g_rows.to(device)).sum().backward()
    t64 = tokens.double().requires_grad_(True)
    o_perm, _, _ = O.permute_routing_map(t64, rmap, probs.double(), num_out_tokens=n, drop_and_pad=True)
    (o_perm * g_rows.double()).sum().backward()
    assert rel_l2(tok_d.grad, t64.grad) <= TOL[dtype]

    # unpermute in the same mode
    rows = torch.randn(n, H, generator=gen).to(dtype)
    g_out = torch.randn(T, H, generator=gen).to(dtype)
    rows_d = rows.to(device).requires_grad_(True)
    probs_u = probs.to(device).requires_grad_(True)
    out = M.unpermute(rows_d, sidx, tokens.shape, probs=probs_u, routing_map=rmap.to(device), fused=True,
                      drop_and_pad=True)
    out.backward(g_out.to(device))
    torch.cuda.synchronize()
    r64 = rows.double().requires_grad_(True)
    p64 = probs.double().requires_grad_(True)
    exp = O.unpermute_routing_map(r64, exp_idx, tokens.shape, p64, rmap, drop_and_pad=True)
    exp.backward(g_out.double())
    assert rel_l2(out, exp) <= TOL[dtype]
    assert rel_l2(rows_d.grad, r64.grad) <= TOL[dtype]
    assert rel_l2(probs_u.grad, p64.grad) <= TOL[dtype]


def test_full_size_properties(device):
    """Mixtral shape (4096 tokens, 8 experts, top-2, hidden 4096, bf16): size-independent properties."""
    T, E, k, H = 4096, 8, 2, 4096
    say("routing-map full size", T, E, k, H)
    rmap, _ = make_map(T, E, k, 99)
    gen = torch.Generator().manual_seed(5)
    tokens = torch.randn(T, H, generator=gen).to(torch.bfloat16)
    rmap_d, tok_d = rmap.to(device), tokens.to(device)
    probs = torch.where(rmap_d, torch.full((T, E), 0.5, device=device), torch.zeros(T, E, device=device))
    perm, pp, sidx = M.permute(tok_d, rmap_d, probs, fused=True)
    counts = rmap.sum(0)
    assert perm.size(0) == T * k and sidx.numel() == T * k
    # expert-major, token-ascending inside every expert
    s = sidx.cpu()
    off = 0
    for e in range(E):
        seg = s[off:off + int(counts[e])]
        assert torch.equal(seg, torch.nonzero(rmap[:, e]).view(-1))
        off += int(counts[e])
    assert torch.equal(perm, tok_d.index_select(0, sidx))
    assert torch.all(pp == 0.5)
    # round trip: weights 1/k give the tokens back exactly (two equal halves of a bf16 value)
    back = M.unpermute(perm, sidx, tok_d.shape, probs=probs, routing_map=rmap_d, fused=True)
    assert torch.equal(back, tok_d)


@pytest.mark.parametrize("T,E", [(5, 4), (1, 32), (300, 7)])
def test_no_entry_set(T, E, device):
    """A map with no entry set: zero rows out; unpermute hands an empty input straight back, like the
    reference does (mindspeed/te/pytorch/permutation.py:81-83)."""
    say("routing-map empty case", T, E)
    rmap = torch.zeros(T, E, dtype=torch.bool, device=device)
    tokens = torch.randn(T, 16, device=device)
    probs = torch.zeros(T, E, device=device)
    perm, pp, sidx = M.permute(tokens, rmap, probs, fused=True)
    assert perm.shape == (0, 16) and pp.numel() == 0 and sidx.numel() == 0
    back = M.unpermute(perm, sidx, tokens.shape, probs=probs, routing_map=rmap, fused=True)
    assert back.numel() == 0


@pytest.mark.parametrize("T,E,k,H,dtype", [
    (300, 8, 2, 256, torch.bfloat16),      # experts a power of two: one launch
    (300, 6, 2, 264, torch.float32),       # any expert count: two launches
    (257, 5, 3, 70, torch.float16),        # odd hidden: element path
    (300, 900, 2, 32, torch.bfloat16),     # many experts: the sort-based path
])
def test_more_rows_than_set_entries(T, E, k, H, dtype, device):
    """A row count above the number of set mask entries (no read-back of the count): the rows that nothing maps to
    come back as zeros, their probabilities as zeros, and everything in front of them as usual."""
    say("routing-map over-provisioned rows", T, E, k, H, dtype)
    rmap, probs = make_map(T, E, k, seed=T + E)
    tokens = torch.randn(T, H, generator=torch.Generator().manual_seed(1)).to(dtype)
    nnz = int(rmap.sum())
    extra = 77
    poison = torch.full((1 << 22,), float("nan"), device=device)       # whatever the allocator hands out next is NaN
    del poison
    perm, pp, sidx = M.permute(tokens.to(device), rmap.to(device), probs.to(dtype).to(device), num_out_tokens=nnz + extra,
                               fused=True)
    o_perm, o_pp, o_sidx = O.permute_routing_map(tokens, rmap, probs.to(dtype))
    assert perm.shape == (nnz + extra, H)
    assert torch.equal(perm[:nnz].cpu(), o_perm) and torch.equal(pp[:nnz].cpu(), o_pp)
    assert torch.equal(perm[nnz:].cpu(), torch.zeros(extra, H, dtype=dtype))
    assert torch.equal(pp[nnz:].cpu(), torch.zeros(extra, dtype=dtype))


def test_argument_checks(device):
    tokens = torch.randn(4, 8, device=device)
    rmap = torch.ones(4, 2, dtype=torch.bool, device=device)
    with pytest.raises(TypeError):
        M.permute(tokens, rmap.to(torch.int32))
    with pytest.raises(RuntimeError):
        M.permute(tokens, rmap[:3])
    with pytest.raises(ValueError):
        M.permute(tokens, rmap, drop_and_pad=True)
    with pytest.raises(ValueError):
        M.unpermute(torch.randn(8, 8, device=device), torch.zeros(8, dtype=torch.int64, device=device), tokens.shape)
    with pytest.raises(RuntimeError):
        M.permute(tokens.cpu(), rmap.cpu())


def test_row_map_is_remembered_on_the_mask(device):
    """unpermute reuses the row map permute computed as long as it gets the same mask tensor in the same state,
    whatever happened to sorted_indices in between; a changed or different mask is sorted again."""
    T, E, k, H = 256, 8, 2, 64
    rmap, probs = make_map(T, E, k, 123)
    rmap_d, probs_d = rmap.to(device), probs.to(device)
    tokens = torch.randn(T, H, device=device).to(torch.bfloat16)
    perm, _, sidx = M.permute(tokens, rmap_d, probs_d, num_out_tokens=T * k, fused=True)
    assert M._recall_row_map(rmap_d, T * k, False) is not None
    calls = []
    real = M.routing_map_row_maps
    M.routing_map_row_maps = lambda *a, **kw: (calls.append(1), real(*a, **kw))[1]
    try:
        out1 = M.unpermute(perm, sidx.clone(), tokens.shape, probs=probs_d, routing_map=rmap_d, fused=True)
        assert not calls                                     # served from the remembered map
        out2 = M.unpermute(perm, sidx, tokens.shape, probs=probs_d, routing_map=rmap_d.clone(), fused=True)
        assert len(calls) == 1                               # another tensor object: sorted afresh
        rmap_d.logical_or_(rmap_d)                           # in-place op: version counter moves on
        assert M._recall_row_map(rmap_d, T * k, False) is None
        out3 = M.unpermute(perm, sidx, tokens.shape, probs=probs_d, routing_map=rmap_d, fused=True)
        assert len(calls) == 2
    finally:
        M.routing_map_row_maps = real
    assert torch.equal(out1, out2) and torch.equal(out1, out3)


@pytest.mark.parametrize("T,E,k,H,dtype", [(300, 8, 2, 256, torch.bfloat16), (300, 6, 2, 70, torch.float32),
                                           (300, 900, 2, 32, torch.bfloat16)])
def test_unpermute_gradient_has_no_unwritten_rows(T, E, k, H, dtype, device):
    """A row count above the number of set entries: the rows of ``grad_permuted`` that nothing maps to are zeros, not
    whatever the allocator handed out; the mapped rows are the oracle's."""
    say("routing-map unpermute gradient, over-provisioned rows", T, E, k, H, dtype)
    rmap, probs = make_map(T, E, k, seed=T + E + 1)
    probs = probs.to(dtype)
    gen = torch.Generator().manual_seed(3)
    tokens = torch.randn(T, H, generator=gen).to(dtype)
    gy = torch.randn(T, H, generator=gen).to(dtype)
    nnz, extra = int(rmap.sum()), 53
    rd, pd = rmap.to(device), probs.to(device)
    perm, _, sidx = M.permute(tokens.to(device), rd, pd, num_out_tokens=nnz + extra, fused=True)
    for with_probs in (True, False):
        pin = perm.detach().clone().requires_grad_(True)
        poison = torch.full((1 << 22,), float("nan"), device=device)
        del poison
        out = M.unpermute(pin, sidx, tokens.shape, probs=pd if with_probs else None, routing_map=rd, fused=True)
        out.backward(gy.to(device))
        torch.cuda.synchronize()
        assert pin.grad.shape == (nnz + extra, H)
        assert torch.count_nonzero(pin.grad[nnz:]) == 0 and not torch.isnan(pin.grad).any()
        o_perm, _, o_sidx = O.permute_routing_map(tokens, rmap, probs)
        o_in = o_perm.clone().requires_grad_(True)
        O.unpermute_routing_map(o_in, o_sidx, tokens.shape, probs=probs if with_probs else None,
                                routing_map=rmap).backward(gy)
        assert rel_l2(pin.grad[:nnz], o_in.grad) <= TOL[dtype]


def test_unpermute_checks_foreign_sorted_indices(device):
    """``unpermute`` gathers by the map the mask gives.  The index tensor that ``permute`` returned for the mask is
    trusted as it is; any other tensor is compared with that map on the device, and one that names another order
    (which the torch path would follow, unpermute_without_activation.py:54-62) is refused instead of being ignored."""
    T, E, k, H = 200, 8, 2, 64
    rmap, probs = make_map(T, E, k, 321)
    rd, pd = rmap.to(device), probs.to(device)
    tokens = torch.randn(T, H, device=device).to(torch.bfloat16)
    perm, _, sidx = M.permute(tokens, rd, pd, num_out_tokens=T * k, fused=True)
    ref = M.unpermute(perm, sidx, tokens.shape, probs=pd, routing_map=rd, fused=True)
    same = M.unpermute(perm, sidx.clone(), tokens.shape, probs=pd, routing_map=rd, fused=True)   # equal values: accepted
    assert torch.equal(ref, same)
    also = M.unpermute(perm, sidx.to(torch.int32), tokens.shape, probs=pd, routing_map=rd, fused=True)
    assert torch.equal(ref, also)
    swapped = sidx.clone()
    swapped[[0, 1]] = swapped[[1, 0]] if swapped[0] != swapped[1] else swapped[[1, 0]] + 1
    with pytest.raises(ValueError, match="token order"):
        M.unpermute(perm, swapped, tokens.shape, probs=pd, routing_map=rd, fused=True)
    with pytest.raises(ValueError, match="token order"):
        M.unpermute(perm, torch.flip(sidx, [0]), tokens.shape, probs=pd, routing_map=rd.clone(), fused=True)


def test_row_map_memory_follows_the_mask_storage(device):
    """The remembered map is tied to the mask's version counter, storage address, shape and strides: a mask whose
    storage was swapped under the same tensor object (``set_``), which leaves the version counter alone, is sorted
    again."""
    T, E, k, H = 128, 8, 2, 32
    rmap, probs = make_map(T, E, k, 77)
    other, _ = make_map(T, E, k, 78)
    rd, pd = rmap.to(device), probs.to(device)
    tokens = torch.randn(T, H, device=device).to(torch.bfloat16)
    M.permute(tokens, rd, pd, num_out_tokens=T * k, fused=True)
    assert M._recall_row_map(rd, T * k, False) is not None
    version = rd._version
    rd.set_(other.to(device))
    assert rd._version == version or M._recall_row_map(rd, T * k, False) is None
    assert M._recall_row_map(rd, T * k, False) is None
    perm, _, sidx = M.permute(tokens, rd, None, num_out_tokens=T * k, fused=True)
    o_perm, _, o_sidx = O.permute_routing_map(tokens.cpu(), other, None)
    assert torch.equal(perm.cpu(), o_perm) and torch.equal(sidx.cpu(), o_sidx)
