"""GPU parity at the benchmark configurations' full sizes: the Mixtral-shape layer (forward + backward), the DeepSeek-V3-style
local share (Zipf routing with one empty expert) and the fine-grained Qwen-MoE-like layer (64 experts, top-8).

Inputs come from the benchmark's own recipe (mindspeed_amd.workloads), so what is timed is what is checked.
Per configuration:
  * row map, forward order, tokens per expert and the permuted rows: bit-exact against the oracle;
  * the layer output, dX and grad_probs on sampled tokens, and dW1 / dW2 on sampled [rows, columns] blocks of
    sampled experts: against an fp32 CPU evaluation of just those rows and blocks, rounded to bf16 where the
    reference's torch path rounds (every op's output), rel-L2 <= 1e-2;
  * an empty expert's weight-gradient blocks are all zeros (the reference test's empty-group rule,
    tests_extend/unit_tests/ops/cann/test_npu_gmm.py:105-113).
The per-row arithmetic follows mindspeed/fsdp/distributed/expert_parallel/dispatcher.py:93-113 (forward) and
the backward recipes of mindspeed/ops/csrc/cann/gmm.cpp:169-246, npu_moe_token_unpermute.cpp:124-148 and
npu_moe_token_permute.cpp:99-118.
"""
import pytest
import torch

from conftest import rel_l2
from oracle import moe_oracle as O

from layer_rowref import RowRef

from mindspeed_amd.dispatcher import dispatch_mlp_combine
from mindspeed_amd.ops import moe_token_permute_with_aux
from mindspeed_amd.workloads import WORKLOADS, make_inputs

pytestmark = pytest.mark.gpu
TOL = 1e-2


def say(*a):
    print(*a, flush=True)


def _span(gen, extent, width):
    """`width` consecutive indices at a random offset, and the last `width` ones."""
    width = min(width, extent)
    a = int(torch.randint(0, extent - width + 1, (1,), generator=gen))
    return [torch.arange(a, a + width), torch.arange(extent - width, extent)]


@pytest.mark.parametrize("name", ["mixtral", "deepseek", "qwen"])
def test_full_size_config_forward_backward(name, device):
    cfg = WORKLOADS[name]
    T, H, E, K, F = cfg["T"], cfg["H"], cfg["E"], cfg["K"], cfg["F"]
    say("config", name, cfg["desc"])
    x, p, idx, w1, w2, gy = make_inputs(cfg, device)
    ref = RowRef(cfg, x, p, idx, w1, w2, gy)
    counts = ref.counts
    say("rows per expert: min", int(counts.min()), "max", int(counts.max()), "empty", int((counts == 0).sum()),
        "below 64:", int(((counts > 0) & (counts < 64)).sum()))
    if name == "deepseek":
        assert int((counts == 0).sum()) >= 1 and int(counts.max()) > 0.3 * T * K      # the recipe's stress points
    if name == "qwen":
        assert int(((counts > 0) & (counts < 64)).sum()) >= 1

    # ---- integer part: bit-exact --------------------------------------------------------------------------
    permuted, row_id_map, sorted_indices, tpe = moe_token_permute_with_aux(x, idx, num_experts=E)
    torch.cuda.synchronize()
    assert torch.equal(row_id_map.cpu(), O.row_id_map(idx.cpu()))
    assert torch.equal(sorted_indices.cpu().long(), ref.fwd)
    assert torch.equal(tpe.cpu(), counts)
    assert torch.equal(permuted, x[(ref.fwd // K).to(device)])

    # ---- the whole layer, forward + backward --------------------------------------------------------------
    leaves = [t.detach().clone().requires_grad_(True) for t in (x, p, w1, w2)]
    out = dispatch_mlp_combine(leaves[0], idx, leaves[1], (leaves[2], leaves[3]))
    dx, dp, dw1, dw2 = torch.autograd.grad(out, leaves, gy)
    torch.cuda.synchronize()
    assert out.shape == (T, H) and dx.shape == (T, H) and dp.shape == (T, K)
    assert dw1.shape == w1.shape and dw2.shape == w2.shape

    # sampled tokens: random ones, some routed to the largest expert, some to the smallest non-empty ones
    gen = torch.Generator().manual_seed(7)
    tokens = torch.randint(0, T, (16,), generator=gen).tolist()
    big = int(torch.argmax(counts))
    nonempty = torch.nonzero(counts > 0).flatten()
    small = nonempty[torch.argsort(counts[nonempty])[:3]].tolist()
    for e in [big] + small:
        r0, r1 = int(ref.offsets[e]), int(ref.offsets[e + 1])
        picks = sorted({r0, r1 - 1, (r0 + r1) // 2})
        tokens += [int(ref.fwd[r]) // K for r in picks]
    tokens = sorted(set(tokens))
    say("sampled tokens:", len(tokens))
    exp_out, exp_dx, exp_dp = ref.token_refs(tokens)
    tsel = torch.tensor(tokens, device=device)
    assert rel_l2(out[tsel], exp_out) <= TOL
    assert rel_l2(dx[tsel], exp_dx) <= TOL
    assert rel_l2(dp[tsel], exp_dp) <= TOL
    worst = max(rel_l2(out[t], exp_out[i]) for i, t in enumerate(tokens))
    say("worst single-token forward rel-L2", f"{worst:.2e}")
    assert worst <= 2 * TOL

    # sampled weight-gradient blocks of the largest, the smallest and two random non-empty experts
    others = nonempty[torch.randperm(len(nonempty), generator=gen)[:2]].tolist()
    for e in sorted(set([big] + small[:2] + others)):
        for ks, fs, hs in zip(_span(gen, H, 64), _span(gen, F, 32), _span(gen, H, 48)):
            e_gate, e_up, e_w2 = ref.dw_blocks(e, ks, fs, hs)
            ksd, fsd, hsd = ks.to(device), fs.to(device), hs.to(device)
            got_gate = dw1[e][ksd][:, fsd]
            got_up = dw1[e][ksd][:, F + fsd]
            got_w2 = dw2[e][fsd][:, hsd]
            errs = (rel_l2(got_gate, e_gate), rel_l2(got_up, e_up), rel_l2(got_w2, e_w2))
            say(f"expert {e} ({int(counts[e])} rows) dW1 gate/up, dW2 block rel-L2:", " ".join(f"{v:.2e}" for v in errs))
            assert max(errs) <= TOL, (e, errs)
    # an expert without rows gets zero weight gradients, and every block is finite
    for e in torch.nonzero(counts == 0).flatten().tolist():
        assert torch.count_nonzero(dw1[e]) == 0 and torch.count_nonzero(dw2[e]) == 0
    assert bool(torch.isfinite(dw1).all()) and bool(torch.isfinite(dw2).all())
    assert bool(torch.isfinite(dx).all()) and bool(torch.isfinite(out).all())
