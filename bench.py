#!/usr/bin/env python3
"""Benchmark of the per-rank MoE expert path on one MI355X.

A step is one forward + backward pass of a single MoE layer (permute, grouped
matmul, SiLU*gate, grouped matmul, weighted unpermute, and all their
gradients) over one batch of synthetic tokens that is resident in HBM before
the timed region starts.  The default workload is the Mixtral-8x7B-shape layer
(4096 tokens, hidden 4096, 8 experts, top-2, FFN 14336, bf16, fp32
accumulation).  One JSON line is printed.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload mixtral|deepseek|qwen|plumbing]
                    [--no-cpu-baseline]
"""
from __future__ import annotations

import argparse
import contextlib
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}   # dense, published

from mindspeed_amd.workloads import WORKLOADS, make_inputs, make_routing  # noqa: E402

# HBM bytes per launch of each grouped-matmul flavour (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by what the same
# counters read for the plain copy kernel of known size), written by `python -m mindspeed_amd.profile_tools traffic`
# together with the hash of the kernel sources they were measured on.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gmm_hbm_traffic.json")

GEMM_KERNEL_NAMES = {
    "gmm_fwd": "gmm16_fast_kernel<bf16, A reduction-contiguous, B column-contiguous> (forward grouped matmul; one "
               "launch each for fc1 and fc2, averaged)",
    "gmm_dx": "gmm16_fast_kernel<bf16, A reduction-contiguous, B reduction-contiguous> (dX grouped matmul on the "
              "transposed weight view; one launch each for fc1 and fc2, averaged)",
    "gmm_dw": "gmm16_fast_kernel<bf16, A row-contiguous, B column-contiguous> (dW grouped matmul, split on the "
              "reduction dim; one launch each for fc1 and fc2, averaged)",
    "gmm_fwd_swiglu": "gmm16_fast_kernel<bf16, A reduction-contiguous, B column-contiguous, SwiGLU epilogue> (fc1 "
                      "forward grouped matmul, one launch per step)",
    "gmm_dx_swiglu": "gmm16_fast_kernel<bf16, A, B reduction-contiguous, SwiGLU-backward epilogue> (fc2 dX grouped "
                     "matmul, one launch per step)",
}


def measured_traffic(workload, kernel):
    """Bytes per launch from the tracked profile, or None when there is none for this workload / kernel or the kernel
    sources have changed since it was taken."""
    from mindspeed_amd.build import source_hash
    try:
        with open(TRAFFIC_FILE) as fh:
            data = json.load(fh)
    except (OSError, ValueError):
        return None
    if data.get("build") != source_hash():
        return None
    return data.get("bytes_per_launch", {}).get(workload, {}).get(kernel)


IN_LAYER_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "permute_family_in_layer.json")


def measured_in_layer_durations(workload):
    """Kernel durations of the HBM-bound ops inside the layer step as rocprofv3 --kernel-trace read them (the event
    brackets under `kernels` include a few microseconds that are not the kernel), from the tracked summary that
    `python -m mindspeed_amd.profile_tools in-layer` wrote: only if it was measured on the kernel sources as they are
    now, else None."""
    from mindspeed_amd.build import source_hash
    try:
        with open(IN_LAYER_FILE) as fh:
            data = json.load(fh)
    except (OSError, ValueError):
        return None
    if data.get("build") != source_hash():
        return None
    return data.get("kernels", {}).get(workload)


def _cpu_layer_once(cfg, sample, dtype=torch.float32):
    from oracle import moe_oracle as O

    T, H, E, K, F = cfg["T"], cfg["H"], cfg["E"], cfg["K"], cfg["F"]
    sub = dict(cfg, T=sample)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(sample, H, generator=gen).to(dtype).requires_grad_(True)
    w1 = (torch.randn(E, H, 2 * F, generator=gen) * 0.02).to(dtype).requires_grad_(True)
    w2 = (torch.randn(E, F, H, generator=gen) * 0.02).to(dtype).requires_grad_(True)
    gy = torch.randn(sample, H, generator=gen).to(dtype)
    p, idx = make_routing(sub, 0)
    p = p.to(dtype).requires_grad_(True)
    t0 = time.perf_counter()
    out = O.moe_layer(x, idx, p, w1, w2)
    torch.autograd.grad(out, (x, p, w1, w2), gy)
    return time.perf_counter() - t0


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, budget_s=12.0):
    """The CPU oracle (torch restatement of the reference's pure-PyTorch path) timed on this host, fp32,
    forward + backward, on a token sample sized (from a short probe run) to about budget_s of CPU work; then the same
    on one thread with a smaller sample."""
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    T = cfg["T"]
    probe = min(T, 128)
    t_probe = _cpu_layer_once(cfg, probe)          # also warms the thread pool
    sample = int(min(T, max(probe, probe * budget_s / max(t_probe, 1e-3))))
    sample = max(64, (sample // 64) * 64) if sample >= 64 else sample
    dt = _cpu_layer_once(cfg, sample) if sample != probe else _cpu_layer_once(cfg, probe)
    torch.set_num_threads(1)
    one = min(sample, 64)
    dt1 = _cpu_layer_once(cfg, one)
    torch.set_num_threads(threads)
    # the workload's own dtype (bf16 matmuls on the CPU are the slower ones: fp32 above is the fair CPU figure)
    extra = {}
    if cfg["dtype"] == "bf16":
        nb = min(sample, 64)
        dtb = _cpu_layer_once(cfg, nb, torch.bfloat16)
        extra["bf16"] = {"value": round(nb / dtb, 2), "unit": "tokens/s", "cores": threads,
                         "sample": f"{nb} tokens, one forward+backward in bf16 ({dtb:.1f} s)"}
    # the headline shape's forward pass whole, once: nothing extrapolated
    if cfg["dtype"] == "bf16" and T * cfg["H"] * cfg["F"] <= 4096 * 4096 * 14336:
        from oracle import moe_oracle as O
        gen = torch.Generator().manual_seed(0)
        H, E, F = cfg["H"], cfg["E"], cfg["F"]
        xw = torch.randn(T, H, generator=gen)
        # only the time is taken: the weights are a random block tiled to the full shape (drawing 1.4 G normal
        # variates on one thread would take longer than the pass itself)
        w1 = torch.randn(1, H, 2 * F // 8, generator=gen).mul_(0.02).repeat(E, 1, 8)
        w2 = torch.randn(1, F // 8, H, generator=gen).mul_(0.02).repeat(E, 8, 1)
        pw, idxw = make_routing(cfg, 0)
        times = []
        with torch.no_grad():
            for _ in range(5):
                t0 = time.perf_counter()
                O.moe_layer(xw, idxw, pw.float(), w1, w2)
                times.append(time.perf_counter() - t0)
                if sum(times) > 25.0:          # a slow host: what has been run so far has to do
                    break
        del xw, w1, w2
        dtw = sorted(times)[len(times) // 2]
        extra["whole_forward"] = {"value": round(T / dtw, 1), "unit": "tokens/s", "cores": threads,
                                  "sample": f"all {T} tokens of the workload, forward pass only (configs[1]), fp32, "
                                            f"median of {len(times)} runs ({dtw:.1f} s): no extrapolation"}
    # configs[0], the reference's CPU-runnable case, whole (no extrapolation): median of five runs
    from mindspeed_amd.workloads import WORKLOADS
    small = WORKLOADS["plumbing"]
    _cpu_layer_once(small, small["T"])
    runs = sorted(_cpu_layer_once(small, small["T"]) for _ in range(5))
    extra["plumbing_config"] = {"value": round(small["T"] / runs[2], 1), "unit": "tokens/s", "cores": threads,
                                "sample": f"{small['desc']}, forward+backward, median of 5 runs ({runs[2] * 1e3:.1f} ms)"}
    return {"value": round(sample / dt, 2), "unit": "tokens/s", "cores": threads, "kind": "port", **extra,
            "sample": f"{sample} of {T} tokens (extrapolated: every expert still reads its whole fp32 weights for that "
                      f"few rows, which is pessimistic for the CPU), same layer shape, fp32, one forward+backward "
                      f"({dt:.1f} s) with torch {torch.__version__} on {threads} threads",
            "single_thread": {"value": round(one / dt1, 2), "unit": "tokens/s", "cores": 1,
                              "sample": f"{one} tokens, one forward+backward ({dt1:.1f} s)"},
            "cpu_model": _cpu_model(), "host_cores": os.cpu_count()}


@contextlib.contextmanager
def threads_on_one_core():
    """Confine every thread of this process to one core for the duration.  The host work of an eager step is serial —
    the main thread issues the forward pass, then waits while torch's autograd thread issues the backward pass — so
    nothing is lost, and the core never goes idle between the two hand-overs of a step.  With the threads on different
    cores each hand-over wakes an idle core, which on these hosts costs about 70 us: the small configuration's step
    reads 0.43-0.45 ms that way and 0.29-0.32 ms on one core (whichever placement the scheduler picks decides the
    figure otherwise: runs of the same loop switch between the two)."""
    saved = {}
    for name in os.listdir("/proc/self/task"):
        try:
            saved[int(name)] = os.sched_getaffinity(int(name))
        except OSError:
            pass
    core = {min(os.sched_getaffinity(0))}
    try:
        for tid in saved:
            try:
                os.sched_setaffinity(tid, core)
            except OSError:
                pass
        yield
    finally:
        for tid, mask in saved.items():
            try:
                os.sched_setaffinity(tid, mask)
            except OSError:
                pass


def measure_routing_map_mode(cfg, device, x, idx, p, iters=200, warmup=20):
    """The routing-map (mask) form of permute / unpermute on the same workload: event-timed averages of the
    forward and of forward+backward, with the algorithmic bytes of the row movement.  Not part of `value`."""
    from mindspeed_amd.ops import moe_permute_mask_map as M

    T, H, E, K = cfg["T"], cfg["H"], cfg["E"], cfg["K"]
    rmap = torch.zeros(T, E, dtype=torch.bool, device=device)
    rmap.scatter_(1, idx, True)
    rows = int(rmap.sum().item())
    probs = torch.zeros(T, E, dtype=torch.float32, device=device).scatter_(1, idx, p.float())
    elem = x.element_size()
    xg = x.detach().clone().requires_grad_(True)
    pg = probs.clone().requires_grad_(True)
    perm, _, sidx = M.permute(xg, rmap, pg, num_out_tokens=rows, fused=True)
    rg = perm.detach().clone().requires_grad_(True)
    g_rows, g_out = torch.randn_like(perm), torch.randn_like(x)

    def timed(fn):
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    def permute_fb():
        out, _, _ = M.permute(xg, rmap, pg, num_out_tokens=rows, fused=True)
        torch.autograd.grad(out, xg, g_rows)

    def unpermute_fb():
        out = M.unpermute(rg, sidx, x.shape, probs=pg, routing_map=rmap, fused=True)
        torch.autograd.grad(out, (rg, pg), g_out)

    t_pf = timed(lambda: M.permute(x, rmap, probs, num_out_tokens=rows, fused=True))
    t_pfb = timed(permute_fb)
    t_uf = timed(lambda: M.unpermute(perm.detach(), sidx, x.shape, probs=probs, routing_map=rmap, fused=True))
    t_ufb = timed(unpermute_fb)
    move = (T + rows) * H * elem       # rows read once + rows written once, either direction
    return {
        "note": "routing-map (mask) form on the same routing; event-timed loops of single ops, host launch "
                "overhead included",
        "rows": rows,
        "permute_fwd": {"avg_ms": round(t_pf, 5), "gbs": round(move / t_pf / 1e6, 1)},
        "permute_fwd_bwd": {"avg_ms": round(t_pfb, 5), "gbs": round(2 * move / t_pfb / 1e6, 1)},
        "unpermute_fwd": {"avg_ms": round(t_uf, 5), "gbs": round(move / t_uf / 1e6, 1)},
        "unpermute_fwd_bwd": {"avg_ms": round(t_ufb, 5), "gbs": round((move + (T + 2 * rows) * H * elem) / t_ufb / 1e6, 1)},
    }


def run_layer(cfg, device, steps, warmup, fuse_activation=False, per_kernel=True, accumulate=None):
    """`warmup` untimed steps, exactly `steps` timed ones between two synchronisations, then (per_kernel) the same
    steps again with every op bracketed by two events on its launch stream.  Returns (ms per step, ms per step with
    the event brackets or None, per-kernel table or None, the inputs).
    accumulate: None, or how the weight gradients reach fp32 `main_grad` buffers of the weights: "fused" = added by
    the weight-gradient product itself (gemm_fusion), "separate" = 16-bit weight gradients and one torch add each."""
    from mindspeed_amd import flop_counter
    from mindspeed_amd.dispatcher import dispatch_mlp_combine

    x, p, idx, w1, w2, gy = make_inputs(cfg, device)
    leaves = [t.requires_grad_(True) for t in (x, p, w1, w2)]
    if accumulate is not None:
        for w in (w1, w2):
            w.main_grad = torch.zeros(w.shape, dtype=torch.float32, device=device)
            w.grad_added_to_main_grad = False

    def step():
        out = dispatch_mlp_combine(leaves[0], idx, leaves[1], (leaves[2], leaves[3]), fuse_activation=fuse_activation,
                                   gemm_fusion=accumulate == "fused")
        grads = torch.autograd.grad(out, leaves, gy)
        if accumulate == "separate":
            w1.main_grad.add_(grads[2])
            w2.main_grad.add_(grads[3])
        return grads

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # timed region: exactly `steps` steps, nothing else on the stream
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    if not per_kernel:
        return ms_per_step, None, None, (x, p, idx)

    with flop_counter.record(timing=True) as rec:
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        ms_events = (time.perf_counter() - t0) * 1e3 / steps
    peak = MFMA_PEAK_TFLOPS[cfg["dtype"]]
    kernels = {}
    for name, s in rec.summary().items():
        avg_ms = s["ms"] / s["calls"]
        work = s["work"] / s["calls"]
        entry = {"calls_per_step": s["calls"] / steps, "avg_ms": round(avg_ms, 5),
                 "ms_per_step": round(s["ms"] / steps, 5)}
        if s["unit"] == "flop":
            entry["tflops"] = round(work / (avg_ms * 1e-3) / 1e12, 2)
            entry["flop_per_launch"] = work
            entry["frac_of_mfma_peak"] = round(entry["tflops"] / peak, 4)
        else:
            entry["gbs"] = round(work / (avg_ms * 1e-3) / 1e9, 1)
            entry["bytes_per_launch"] = work
            entry["frac_of_hbm_peak"] = round(entry["gbs"] / HBM_PEAK_GBS, 4)
        kernels[name] = entry
    return ms_per_step, ms_events, kernels, (x, p, idx)


def forward_only_ms(cfg, device, fuse_activation, steps=20, warmup=10):
    """The layer's forward pass alone under ``torch.no_grad()`` (inference): ms per pass.  With ``fuse_activation`` the
    SwiGLU comes out of the first grouped matmul's epilogue and the fc1 output, which only a backward pass would read,
    is not stored."""
    from mindspeed_amd.dispatcher import dispatch_mlp_combine

    x, p, idx, w1, w2, _ = make_inputs(cfg, device)
    with torch.no_grad():
        for _ in range(warmup):
            dispatch_mlp_combine(x, idx, p, (w1, w2), fuse_activation=fuse_activation)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            dispatch_mlp_combine(x, idx, p, (w1, w2), fuse_activation=fuse_activation)
        torch.cuda.synchronize()
    return round((time.perf_counter() - t0) * 1e3 / steps, 4)


def graph_replay_ms(cfg, device, replays=200):
    """One forward+backward step of the layer recorded into a HIP graph (the C ABI only launches kernels on the
    caller's stream, so the step can be captured) and replayed: ms per replay, or None if a replay does not reproduce
    the eager step bit for bit.  For the small configuration, whose eager step time is the host's launch work."""
    from mindspeed_amd.dispatcher import dispatch_mlp_combine

    x, p, idx, w1, w2, gy = make_inputs(cfg, device)

    def step():
        leaves = [t.detach().requires_grad_(True) for t in (x, p, w1, w2)]
        out = dispatch_mlp_combine(leaves[0], idx, leaves[1], (leaves[2], leaves[3]))
        return (out,) + tuple(torch.autograd.grad(out, leaves, gy))

    eager = [t.clone() for t in step()]
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(device)
    side.wait_stream(torch.cuda.current_stream(device))
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph):
            outs = step()
    torch.cuda.current_stream(device).wait_stream(side)
    torch.cuda.synchronize()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    if not all(torch.equal(a, b) for a, b in zip(outs, eager)):
        return None
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    return round((time.perf_counter() - t0) * 1e3 / replays, 4)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="mixtral", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="only the timed steps and the per-kernel table (no other workloads, no permute-family or "
                         "routing-map sections)")
    ap.add_argument("--fuse-activation", action="store_true",
                    help="run the expert MLP with SwiGLU fused into the neighbouring grouped matmuls "
                         "(default: the reference's op sequence, one kernel per op)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="after the steps, run the plain copy kernel over this many MiB three times "
                         "(reference point for profiler byte counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one rank's expert path on ONE GPU (no collectives are part of this path); "
                 "run it with --gpus 1.")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")

    cfg = WORKLOADS[args.workload]
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    ms_per_step, ms_per_step_events, kernels, (x, p, idx) = run_layer(
        cfg, device, args.steps, args.warmup, args.fuse_activation)
    tokens_per_s = cfg["T"] / (ms_per_step / 1e3)

    # what an empty bracket reads: the per-op times include this much that is not the kernel
    stream = torch.cuda.current_stream(device)
    pairs = []
    for _ in range(50):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        e1.record(stream)
        pairs.append((e0, e1))
    torch.cuda.synchronize()
    empty_bracket_ms = sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)

    # dominant kernel: the grouped-matmul flavour with the largest share of the step
    peak = MFMA_PEAK_TFLOPS[cfg["dtype"]]
    gemms = {k: v for k, v in kernels.items() if "tflops" in v}
    dom_name = max(gemms, key=lambda k: gemms[k]["ms_per_step"])
    dom = gemms[dom_name]
    kname = GEMM_KERNEL_NAMES.get(dom_name, dom_name) if cfg["dtype"] == "bf16" else \
        f"gmm32_kernel ({dom_name}, fp32 inputs)"
    roofline = {"bound": "mfma", "kernel": kname, "kernel_key": dom_name,
                "share_of_step": round(dom["ms_per_step"] / sum(v["ms_per_step"] for v in kernels.values()), 4),
                "achieved": dom["tflops"], "peak": peak, "unit": "TFLOP/s", "frac": dom["frac_of_mfma_peak"],
                "traffic": measured_traffic(args.workload, dom_name)}

    result = {
        "metric": "MoE layer fwd+bwd tokens/s at 1 GPU",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_with_event_timing": round(ms_per_step_events, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": cfg["desc"], "tokens": cfg["T"], "hidden": cfg["H"], "experts": cfg["E"],
                   "topk": cfg["K"], "ffn": cfg["F"], "fused_activation": bool(args.fuse_activation),
                   "gemm_tflop_per_step": round(18.0 * cfg["T"] * cfg["K"] * cfg["H"] * cfg["F"] / 1e12, 3)},
        "roofline": roofline,
        "kernels": kernels,
        "kernels_note": "single launches inside the layer step, each between two events on its stream; an empty "
                        f"bracket reads {empty_bracket_ms * 1e3:.1f} us on this box",
    }
    if args.copy_calibration:
        from mindspeed_amd import microbench_kernels
        n = args.copy_calibration << 20
        src = torch.empty(n, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            microbench_kernels.copy_bytes(src, dst)
        torch.cuda.synchronize()
        result["copy_calibration_bytes"] = n
    def extra(name, fn):
        """Sections beside the headline measurement: one that raises is reported under `extras_failed` and the line
        is printed all the same."""
        try:
            fn()
        except Exception as exc:      # noqa: BLE001 -- whatever it is, the measured line must still come out
            import traceback
            traceback.print_exc(file=sys.stderr)
            result.setdefault("extras_failed", {})[name] = repr(exc)
        torch.cuda.empty_cache()

    def routing_map_section():
        result["routing_map_mode"] = measure_routing_map_mode(cfg, device, x.detach(), idx, p.detach())
        # these loops are host-bound too, and the forward+backward ones hand over to the autograd thread
        with threads_on_one_core():
            pinned = measure_routing_map_mode(cfg, device, x.detach(), idx, p.detach())
        result["routing_map_mode"]["avg_ms_threads_on_one_core"] = {
            k: v["avg_ms"] for k, v in pinned.items() if isinstance(v, dict)}

    def permute_family_section():
        # The permute / unpermute family by itself at this workload's shape: back-to-back launches through the C ABI
        # (the per-op figures under "kernels" are single launches inside the layer step, whose operands were last
        # touched hundreds of megabytes of traffic earlier).  "warm": one set of buffers, resident in the 256 MB
        # last-level cache at this size; "cold": launches rotate through enough buffer sets to exceed that cache
        # six times, so every launch streams from HBM.  Not part of `value`.
        from mindspeed_amd.permute_microbench import measure as measure_permute_family, sets_for_cold
        shape = (cfg["T"], cfg["H"], cfg["E"], cfg["K"], torch.bfloat16)
        cold_sets = sets_for_cold(cfg["T"], cfg["H"], cfg["K"])
        warm = measure_permute_family(*shape, device=device)
        cold = measure_permute_family(*shape, device=device, sets=cold_sets)
        for table in (warm, cold):
            for r in table.values():
                r["frac_of_copy"] = round(r["gbs"] / table["copy"]["gbs"], 3)
        result["permute_family"] = {
            "note": "back-to-back launches through the C ABI, event-timed over 200 launches per op; algorithmic bytes "
                    "over the average, against the 8 TB/s HBM peak and against the plain copy kernel in the same mode",
            "cold_buffer_sets": cold_sets, "warm": warm, "cold": cold}
        if args.workload == "mixtral":
            # the same at the shapes of the other two benchmark configurations (index form and routing-map form of the
            # four ops, and the copy), fraction of the 8 TB/s peak and of the copy: their buffers exceed the
            # last-level cache already with one set, the rotation ("cold") adds a second or third
            brief = ("permute", "permute_mask", "unpermute", "unpermute_mask", "unpermute_grad", "permute_grad", "copy")
            for name in ("deepseek", "qwen"):
                o = WORKLOADS[name]
                oshape = (o["T"], o["H"], o["E"], o["K"], torch.bfloat16)
                tables = {"one_buffer_set": measure_permute_family(*oshape, device=device, iters=100),
                          "cold": measure_permute_family(*oshape, device=device, iters=100,
                                                         sets=sets_for_cold(o["T"], o["H"], o["K"]))}
                result["permute_family"][name] = {
                    "shape": f"{o['T']} tokens x hidden {o['H']}, {o['E']} experts, top-{o['K']}",
                    **{mode: {k: {"avg_us": t[k]["avg_us"], "frac_of_hbm_peak": t[k]["frac_of_hbm_peak"],
                                  "frac_of_copy": round(t[k]["gbs"] / t["copy"]["gbs"], 3)} for k in brief}
                       for mode, t in tables.items()}}
                torch.cuda.empty_cache()
        in_layer = measured_in_layer_durations(args.workload)
        if in_layer is not None:
            result["permute_family"]["in_layer_rocprofv3"] = in_layer

    others = {}

    def other_workload(name):
        # forward+backward, 10 steps after its own warm-up; the small one, whose step is a third of a millisecond of
        # host work, needs 100 steps until the host side (allocator, caches) has settled and is timed over 300
        ocfg = WORKLOADS[name]
        small = name == "plumbing"
        ms, _, ok, _ = run_layer(ocfg, device, steps=300 if small else 10, warmup=100 if small else 10)
        others[name] = {"workload": ocfg["desc"], "ms_per_step": round(ms, 4),
                        "tokens_per_s": round(ocfg["T"] / (ms / 1e3), 1),
                        "gemm_tflops": {k: ok[k]["tflops"] for k in ("gmm_fwd", "gmm_dx", "gmm_dw") if k in ok},
                        "gemm_frac_of_mfma_peak": {k: ok[k]["frac_of_mfma_peak"]
                                                   for k in ("gmm_fwd", "gmm_dx", "gmm_dw") if k in ok}}
        if small:
            # the same steps with the process's threads on one core (see threads_on_one_core)
            with threads_on_one_core():
                ms1, _, _, _ = run_layer(ocfg, device, steps=300, warmup=100, per_kernel=False)
            others[name]["ms_per_step_threads_on_one_core"] = round(ms1, 4)
            others[name]["note"] = ("ms_per_step: threads placed by the scheduler; the step is host-bound and reads "
                                    "0.27-0.45 ms depending on whether the main and the autograd thread share a core")

    def graph_section():
        others["plumbing"]["graph_replay_ms_per_step"] = graph_replay_ms(WORKLOADS["plumbing"], device)

    def accumulation_section():
        # the same Mixtral step with the weight gradients accumulated into fp32 buffers (the reference's
        # gradient-accumulation fusion, mindspeed/ops/gmm.py:56-89) by the product itself, against 16-bit
        # weight gradients followed by one add each
        acc = {}
        for how in ("fused", "separate"):
            ms, _, ok, _ = run_layer(cfg, device, steps=10, warmup=5, accumulate=how)
            acc[how] = {"ms_per_step": round(ms, 4),
                        "gmm_dw_tflops": ok["gmm_dw"]["tflops"] if "gmm_dw" in ok else None}
            torch.cuda.empty_cache()
        others["mixtral_fp32_grad_accumulation"] = acc

    def forward_only_section():
        others["mixtral_forward_only"] = {
            "note": "forward pass alone under torch.no_grad(), ms per pass and tokens/s",
            **{name: {"ms": ms, "tokens_per_s": round(cfg["T"] / (ms / 1e3), 1)}
               for name, ms in (("one_kernel_per_op", forward_only_ms(cfg, device, False)),
                                ("fused_activation", forward_only_ms(cfg, device, True)))}}

    if not args.no_extras:
        extra("routing_map_mode", routing_map_section)
        extra("permute_family", permute_family_section)
        if args.workload == "mixtral":
            del x, p, idx
            torch.cuda.empty_cache()
            for name in ("deepseek", "qwen", "plumbing"):
                extra(name, lambda name=name: other_workload(name))
            if "plumbing" in others:
                extra("plumbing_graph_replay", graph_section)
            extra("mixtral_fp32_grad_accumulation", accumulation_section)
            extra("mixtral_forward_only", forward_only_section)
            result["other_workloads"] = others
    if not args.no_cpu_baseline:
        extra("cpu_baseline", lambda: result.__setitem__("cpu_baseline", cpu_baseline(cfg)))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
