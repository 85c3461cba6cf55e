"""Synthetic workloads of the per-rank MoE expert path: shapes, routing recipes and input tensors.

One recipe serves the benchmark and the full-size GPU parity tests, so both see the same bits.  Routing is
generated on the CPU from a seeded generator (identical on every host); activations and weights on the device.
"""
from __future__ import annotations

import torch

WORKLOADS = {
    # name: tokens T, hidden H, experts E, top-k K, expert FFN F, dtype, routing recipe
    "plumbing": dict(T=512, H=256, E=8, K=2, F=512, dtype="f32", routing="uniform",
                     desc="configs[0]: 512 tokens, hidden 256, 8 experts, top-2, ffn 512, fp32"),
    "mixtral": dict(T=4096, H=4096, E=8, K=2, F=14336, dtype="bf16", routing="uniform",
                    desc="configs[1]/[2] Mixtral-8x7B-shape MoE layer: 4096 tokens, hidden 4096, 8 experts, "
                         "top-2, ffn 14336, bf16, forward+backward"),
    "deepseek": dict(T=2048, H=7168, E=8, K=8, F=2048, dtype="bf16", routing="zipf_empty",
                     desc="configs[3] DeepSeek-V3-style local share: 16384 rows, hidden 7168, 8 local experts, "
                          "ffn 2048, Zipf(1.2) with one empty expert, bf16, forward+backward"),
    "qwen": dict(T=8192, H=2048, E=64, K=8, F=1408, dtype="bf16", routing="biased",
                 desc="configs[4] fine-grained MoE: 8192 tokens, hidden 2048, 64 experts, top-8, ffn 1408, "
                      "biased routing, bf16, forward+backward"),
}


def make_routing(cfg, seed=0):
    """Routing probabilities ``[T, K]`` (fp32) and expert indices ``[T, K]`` (int64) on the CPU.

    ``uniform``: logits ~ N(0,1), softmax, top-k, renormalised.  ``biased``: the same with a per-expert bias
    ~ N(0, 1.5).  ``zipf_empty``: every (token, slot) row draws its expert from Zipf(1.2) over the shuffled
    experts, one expert is forced empty (its rows go to the next expert), probabilities ~ Dirichlet(1) per token.
    """
    gen = torch.Generator().manual_seed(seed)
    T, E, K = cfg["T"], cfg["E"], cfg["K"]
    if cfg["routing"] == "zipf_empty":
        pmf = 1.0 / torch.arange(1, E + 1, dtype=torch.float64) ** 1.2
        pmf = pmf[torch.randperm(E, generator=gen)]
        empty = int(torch.randint(0, E, (1,), generator=gen))
        idx = torch.multinomial(pmf / pmf.sum(), T * K, replacement=True, generator=gen)
        idx[idx == empty] = (empty + 1) % E
        idx = idx.view(T, K)
        probs = torch.distributions.Dirichlet(torch.ones(K)).sample((T,))
        return probs.float(), idx
    logits = torch.randn(T, E, generator=gen)
    if cfg["routing"] == "biased":
        logits = logits + 1.5 * torch.randn(E, generator=gen)
    full = torch.softmax(logits, dim=-1)
    p, idx = torch.topk(full, K, dim=-1)
    return (p / p.sum(-1, keepdim=True)).float(), idx


def make_inputs(cfg, device, seed=0):
    """``(x [T,H], probs [T,K], indices [T,K], w_gate_up [E,H,2F], w_down [E,F,H], dY [T,H])`` on ``device``:
    x, dY ~ N(0,1), weights ~ N(0, 0.02), in the workload's dtype."""
    dtype = torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float32
    T, H, E, F = cfg["T"], cfg["H"], cfg["E"], cfg["F"]
    gen = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(T, H, generator=gen, device=device).to(dtype)
    w1 = (torch.randn(E, H, 2 * F, generator=gen, device=device) * 0.02).to(dtype)
    w2 = (torch.randn(E, F, H, generator=gen, device=device) * 0.02).to(dtype)
    gy = torch.randn(T, H, generator=gen, device=device).to(dtype)
    p, idx = make_routing(cfg, seed)
    return x, p.to(dtype).to(device), idx.to(device), w1, w2, gy
