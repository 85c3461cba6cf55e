"""Grouped-matmul launches of the Mixtral-shape expert MLP in isolation.

    python -m mindspeed_amd.gmm_microbench [--mode fwd1|fwd2|dx1|dx2|dw1|dw2|dw1acc|dw2acc|library|all]
                                           [--data randn|small|ones|zeros]
                                           [--dtype bf16|fp16|fp32] [--counts 988,1074,...] [--iters 20] [--warmup 20]

``fwd1`` / ``dx1`` / ``dw1`` are the forward, dX and dW products of the first matmul
(``[T, H] x [E, H, 2F]``), ``fwd2`` / ``dx2`` / ``dw2`` those of the second (``[T, F] x [E, F, H]``);
``dw1acc`` / ``dw2acc`` are the weight gradients added in place to an fp32 buffer;
``library`` runs ``torch.bmm`` on the fc1-forward shape as E dense products, for orientation (contiguous operands
only: a run of this program's loop with ``torch.bmm`` on transposed views of these shapes ended in a GPU memory fault
inside the vendor library's launches, so those layouts are not offered).  ``all`` launches the six products one after the other,
``--iters`` launches each and no warm-up, in the fixed order fwd1 fwd2 dx1 dx2 dw1 dw2: the form to put under
``rocprofv3 --pmc`` (``python -m mindspeed_amd.profile_tools products`` reads the counters back per product).
``--data`` sets the operand values only (the rate of the matrix cores on this board depends on them);
``--counts`` gives the rows per expert (default: equal shares).  Prints milliseconds per launch and TFLOP/s.
"""
from __future__ import annotations

import argparse

import torch

from .ops.gmm import gmm_raw


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--mode", default="fwd1", choices=["fwd1", "fwd2", "dx1", "dx2", "dw1", "dw2", "dw1acc", "dw2acc", "library", "all"])
    ap.add_argument("--data", default="randn", choices=["randn", "small", "ones", "zeros"])
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16", "fp32"], help="operand dtype")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8192, help="rows after permutation (tokens x top-k)")
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--ffn", type=int, default=14336)
    ap.add_argument("--experts", type=int, default=8)
    ap.add_argument("--counts", default="", help="comma-separated rows per expert (must sum to --tokens)")
    a = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("needs a HIP device")
    dev = torch.device("cuda", 0)
    T, H, F, E = a.tokens, a.hidden, a.ffn, a.experts
    gen = torch.Generator(device=dev).manual_seed(0)
    if a.counts:
        counts = torch.tensor([int(v) for v in a.counts.split(",")], dtype=torch.int64, device=dev)
        if counts.numel() != E or int(counts.sum()) != T:
            raise SystemExit(f"--counts needs {E} entries summing to {T}")
    else:
        counts = torch.full((E,), T // E, dtype=torch.int64, device=dev)
    bf = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[a.dtype]

    def operand(*shape):
        if a.data == "zeros":
            return torch.zeros(*shape, device=dev, dtype=bf)
        if a.data == "ones":
            return torch.ones(*shape, device=dev, dtype=bf)
        if a.data == "small":
            return torch.randint(-2, 3, shape, generator=gen, device=dev).to(bf)
        return torch.randn(*shape, generator=gen, device=dev).to(bf)

    if a.mode == "all":
        x1, w1, dy1 = operand(T, H), operand(E, H, 2 * F), operand(T, 2 * F)
        x2, w2, dy2 = operand(T, F), operand(E, F, H), operand(T, H)
        products = [("fwd1", lambda: gmm_raw(x1, w1, counts, 0, 1)), ("fwd2", lambda: gmm_raw(x2, w2, counts, 0, 1)),
                    ("dx1", lambda: gmm_raw(dy1, w1.transpose(1, 2), counts, 0, 1)),
                    ("dx2", lambda: gmm_raw(dy2, w2.transpose(1, 2), counts, 0, 1)),
                    ("dw1", lambda: gmm_raw(x1.t(), dy1, counts, 2, 1)), ("dw2", lambda: gmm_raw(x2.t(), dy2, counts, 2, 1))]
        torch.cuda.synchronize()
        for name, fn in products:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(a.iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            print(f"{name} ({a.data}): {e0.elapsed_time(e1) / a.iters:.4f} ms per launch over {a.iters} launches", flush=True)
        return
    if a.mode == "fwd1":
        x, w = operand(T, H), operand(E, H, 2 * F)
        fn, flops = (lambda: gmm_raw(x, w, counts, 0, 1)), 2 * T * H * 2 * F
    elif a.mode == "fwd2":
        x, w = operand(T, F), operand(E, F, H)
        fn, flops = (lambda: gmm_raw(x, w, counts, 0, 1)), 2 * T * H * F
    elif a.mode == "dx1":
        dy, w = operand(T, 2 * F), operand(E, H, 2 * F)
        fn, flops = (lambda: gmm_raw(dy, w.transpose(1, 2), counts, 0, 1)), 2 * T * H * 2 * F
    elif a.mode == "dx2":
        dy, w = operand(T, H), operand(E, F, H)
        fn, flops = (lambda: gmm_raw(dy, w.transpose(1, 2), counts, 0, 1)), 2 * T * H * F
    elif a.mode == "dw1":
        x, dy = operand(T, H), operand(T, 2 * F)
        fn, flops = (lambda: gmm_raw(x.t(), dy, counts, 2, 1)), 2 * T * H * 2 * F
    elif a.mode == "dw2":
        x, dy = operand(T, F), operand(T, H)
        fn, flops = (lambda: gmm_raw(x.t(), dy, counts, 2, 1)), 2 * T * H * F
    elif a.mode in ("dw1acc", "dw2acc"):
        # the fp32 `+=` form of the weight gradient (npu_groupmatmul_add_fp32): the sums grow by one product per
        # launch, which leaves fp32 range only after ~1e30 launches
        x, dy = (operand(T, H), operand(T, 2 * F)) if a.mode == "dw1acc" else (operand(T, F), operand(T, H))
        grad = torch.zeros(E, x.size(1), dy.size(1), device=dev, dtype=torch.float32)
        fn, flops = (lambda: gmm_raw(x.t(), dy, counts, 2, 1, out=grad, accumulate=True)), 2 * T * x.size(1) * dy.size(1)
    else:
        x, w = operand(E, T // E, H), operand(E, H, 2 * F)
        fn, flops = (lambda: torch.bmm(x, w)), 2 * T * H * 2 * F
    for _ in range(a.warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(a.iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / a.iters
    print(f"{a.mode} ({a.data}{'' if a.dtype == 'bf16' else ', ' + a.dtype}): {ms:.4f} ms  {flops / ms / 1e9:.1f} TFLOP/s", flush=True)


if __name__ == "__main__":
    main()
