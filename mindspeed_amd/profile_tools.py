"""Measurement helpers behind the figures under ``profiles/``.

    python -m mindspeed_amd.profile_tools traffic --fetch F.csv --write W.csv [--workload mixtral] [--out FILE.json]
    python -m mindspeed_amd.profile_tools counters [--all] CSV [CSV ...]
    python -m mindspeed_amd.profile_tools in-layer --stats KERNEL_STATS.csv [--workload mixtral] [--out FILE.json]
    python -m mindspeed_amd.profile_tools products --csv COUNTERS.csv [--iters 3]
    python -m mindspeed_amd.profile_tools power [--seconds 4] [--modes fwd1,dx1,dw1] [--data randn,zeros]
    MINDSPEED_AMD_LIB=mindspeed_amd/libmindspeed_amd_trace.so python -m mindspeed_amd.profile_tools timeline [--modes ...] [--data ...]

``traffic`` reads the ``*_counter_collection.csv`` files of two ``rocprofv3 --pmc`` runs of ``bench.py`` (one with
FETCH_SIZE, one with WRITE_SIZE; both with ``--copy-calibration MIB`` so that the plain copy kernel of known size is
among the dispatches), scales the counters by what they read for that copy, prints HBM bytes per dispatch for every
kernel of the library and, with ``--out``, records the grouped-matmul figures together with the hash of the kernel
sources they belong to (``bench.py`` reports them as ``roofline.traffic`` as long as that hash is unchanged).

``counters`` prints per-kernel averages of whatever counters the given files hold (this library's kernels only) and
the ratios derived from them: MFMA busy share, LDS-wait and any-wait share of the wavefront cycles, LDS bank conflicts
per LDS instruction cycle, L2 hit rate.

``in-layer`` turns the kernel statistics of a ``rocprofv3 --kernel-trace --stats`` run of ``bench.py`` into the
durations and HBM-roofline fractions of the permute / unpermute / SwiGLU kernels inside the layer step.

``power`` runs one grouped-matmul launch of the Mixtral-shape expert MLP back to back for a few seconds per
(product, operand values) pair while a thread samples the board's power draw and shader clock from the amdgpu
hwmon / sysfs files (read-only), and prints rate, power and clock side by side.

``timeline`` needs the diagnostic build of the library (``python -m mindspeed_amd.build --trace``, selected with
MINDSPEED_AMD_LIB): it launches one grouped matmul of the same shapes, reads the per-workgroup time stamps back and
prints how a tile's time splits into finding the tile, waiting for the first operands, the K loop and the epilogue,
and how long a compute unit stands idle between two workgroups.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import re
import sys
import threading
import time

GEMM_KEYS = {  # first template arguments <dtype, A reduction-contiguous, B reduction-contiguous, output mode, ...>
    "gmm16_fast_kernel<0, true, false, 0,": "gmm_fwd",
    "gmm16_fast_kernel<0, true, true, 0,": "gmm_dx",
    "gmm16_fast_kernel<0, false, false, 0,": "gmm_dw",
    "gmm16_fast_kernel<0, true, false, 3,": "gmm_fwd_swiglu",
    "gmm16_fast_kernel<0, true, true, 4,": "gmm_dx_swiglu",
}


def short_name(name: str) -> str:
    name = name.replace("void ", "").replace("ms::(anonymous namespace)::", "").replace("(anonymous namespace)::", "")
    name = re.sub(r"\(.*$", "", name)
    return name.replace("(ms::OutMode)", "").replace("(int)", "")


def read_counter(path: str, counter: str):
    """kernel -> list of per-dispatch values of `counter`."""
    per_kernel = collections.defaultdict(list)
    with open(path, newline="") as fh:
        for row in csv.DictReader(fh):
            if row["Counter_Name"] == counter:
                per_kernel[short_name(row["Kernel_Name"])].append(float(row["Counter_Value"]))
    return per_kernel


def calibration(per_kernel, known_kib: float):
    """Scale factor of a byte counter from the copy kernel's largest dispatches (a transfer of `known_kib` KiB)."""
    copies = [v for k, vals in per_kernel.items() if "copy_bytes_kernel" in k for v in vals]
    if not copies:
        raise SystemExit("no copy_bytes_kernel dispatches in the counter file: run bench.py with --copy-calibration MIB")
    big = [v for v in copies if v >= 0.9 * max(copies)]
    return known_kib / (sum(big) / len(big)), sum(big) / len(big), len(big)


def cmd_traffic(args):
    from .build import source_hash

    fetch = read_counter(args.fetch, "FETCH_SIZE")
    write = read_counter(args.write, "WRITE_SIZE")
    known_kib = args.copy_mib * 1024.0
    f_scale, f_read, f_n = calibration(fetch, known_kib)
    w_scale, w_read, w_n = calibration(write, known_kib)
    print(f"calibration: {f_n} copy_bytes_kernel dispatches over {args.copy_mib} MiB read FETCH_SIZE = {f_read:.0f}, "
          f"WRITE_SIZE = {w_read:.0f} (KiB moved each way: {known_kib:.0f})")
    print(f"  -> scale factors: FETCH_SIZE x {f_scale:.3f}, WRITE_SIZE x {w_scale:.3f}\n")
    print(f"{'kernel':84s} {'disp':>5s} {'fetch_MB':>10s} {'write_MB':>10s} {'total_MB':>10s}")
    record = {}
    for kernel in fetch:
        if "ms::" not in kernel and "gmm" not in kernel and "kernel" not in kernel:
            continue
        f = fetch[kernel]
        w = write.get(kernel, [])
        if not w:
            continue
        f_mb = sum(f) / len(f) * f_scale * 1024 / 1e6
        w_mb = sum(w) / len(w) * w_scale * 1024 / 1e6
        print(f"{kernel[:84]:84s} {len(f):5d} {f_mb:10.1f} {w_mb:10.1f} {f_mb + w_mb:10.1f}")
        for pattern, key in GEMM_KEYS.items():
            if pattern in kernel:
                record[key] = int(round((f_mb + w_mb) * 1e6))
    if args.out:
        data = {}
        if os.path.exists(args.out):
            with open(args.out) as fh:
                data = json.load(fh)
        build = source_hash()
        if data.get("build") != build:
            data = {"build": build, "unit": "HBM bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by the copy "
                                            "kernel's reading; launches of fc1 and fc2 averaged)", "bytes_per_launch": {}}
        data["bytes_per_launch"][args.workload] = record
        with open(args.out, "w") as fh:
            json.dump(data, fh, indent=1, sort_keys=True)
            fh.write("\n")
        print(f"\nrecorded {record} for build {build} in {args.out}")


def _own_kernel(name: str) -> bool:
    """Kernels of this library (everything else in a trace is torch's own: fills, copies, random numbers)."""
    return not name.startswith(("at::", "__amd", "rocclr")) and "at::native" not in name


def cmd_counters(args):
    """Per-kernel averages of the counters in the given files, this library's kernels only, and below them the ratios
    they are collected for."""
    merged = collections.defaultdict(dict)
    for path in args.files:
        agg = collections.defaultdict(lambda: collections.defaultdict(list))
        with open(path, newline="") as fh:
            for row in csv.DictReader(fh):
                agg[short_name(row["Kernel_Name"])][row["Counter_Name"]].append(float(row["Counter_Value"]))
        print(f"# {os.path.basename(path)}")
        for kernel, counters in agg.items():
            if not _own_kernel(kernel) or (not args.all and "gmm16" not in kernel):
                continue
            for counter, vals in counters.items():
                avg = sum(vals) / len(vals)
                merged[kernel][counter] = avg
                print(f"{kernel[:70]:70s} {counter:28s} dispatches {len(vals):5d}  avg {avg:16.1f}")
    print("\n# derived (averages per dispatch)")
    print(f"{'kernel':70s} {'MFMA busy':>10s} {'LDS wait':>10s} {'any wait':>10s} {'LDS bank confl.':>16s} {'L2 hit rate':>12s}")
    for kernel, c in merged.items():
        def ratio(num, den, scale=1.0):
            return f"{c[num] / (scale * c[den]):.3f}" if num in c and den in c and c[den] else "-"
        hit = f"{c['TCC_HIT_sum'] / (c['TCC_HIT_sum'] + c['TCC_MISS_sum']):.3f}" if "TCC_HIT_sum" in c and "TCC_MISS_sum" in c else "-"
        # SQ_WAVE_CYCLES counts in units of 4 clocks per wavefront, the busy / wait counters in clocks
        print(f"{kernel[:70]:70s} {ratio('SQ_VALU_MFMA_BUSY_CYCLES', 'SQ_WAVE_CYCLES', 4.0):>10s} "
              f"{ratio('SQ_WAIT_INST_LDS', 'SQ_WAVE_CYCLES', 4.0):>10s} {ratio('SQ_WAIT_INST_ANY', 'SQ_WAVE_CYCLES', 4.0):>10s} "
              f"{ratio('SQ_LDS_BANK_CONFLICT', 'SQ_ACTIVE_INST_LDS'):>16s} {hit:>12s}")


def cmd_products(args):
    """Per-product L2 counters of `python -m mindspeed_amd.gmm_microbench --mode all --iters N` run under
    `rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_EA0_RDREQ_sum TCC_EA0_WRREQ_sum`: the grouped-matmul dispatches come in
    the order fwd1 fwd2 dx1 dx2 dw1 dw2, N of each; the first of each product is left out of the average.  Reads from
    the fabric are 128-byte requests (one L2 line), writes 64-byte ones (checked on kernels of known traffic)."""
    rows = collections.OrderedDict()
    with open(args.csv, newline="") as fh:
        for row in csv.DictReader(fh):
            if "gmm16_fast_kernel" in row["Kernel_Name"]:
                rows.setdefault(int(row["Dispatch_Id"]), {})[row["Counter_Name"]] = float(row["Counter_Value"])
    ids = sorted(rows)
    names = ("fwd1", "fwd2", "dx1", "dx2", "dw1", "dw2")
    if len(ids) != len(names) * args.iters:
        raise SystemExit(f"expected {len(names) * args.iters} grouped-matmul dispatches, found {len(ids)}")
    print(f"{'product':8s} {'fabric reads GB':>16s} {'fabric writes GB':>17s} {'L2 hit rate':>12s}")
    for i, name in enumerate(names):
        grp = [rows[j] for j in ids[i * args.iters:(i + 1) * args.iters]][1 if args.iters > 1 else 0:]
        avg = {k: sum(g[k] for g in grp) / len(grp) for k in grp[0]}
        hit = avg["TCC_HIT_sum"] / (avg["TCC_HIT_sum"] + avg["TCC_MISS_sum"])
        print(f"{name:8s} {avg['TCC_EA0_RDREQ_sum'] * 128 / 1e9:16.2f} {avg['TCC_EA0_WRREQ_sum'] * 64 / 1e9:17.2f} {hit:12.3f}")


# kernels of the HBM-bound ops inside the layer step: name fragment -> (label, algorithmic bytes of one launch)
def _in_layer_ops(cfg):
    from . import flop_counter
    T, K, H, F = cfg["T"], cfg["K"], cfg["H"], cfg["F"]
    elem = 2 if cfg["dtype"] == "bf16" else 4
    rows = T * K
    return {
        "permute_fused_kernel": ("permute", flop_counter.permute_bytes(T, K, H, elem, 8)),
        "permute_fused_bins_kernel": ("permute", flop_counter.permute_bytes(T, K, H, elem, 8)),
        "permute_scatter_rows_kernel": ("permute (rows launch; the histogram launch is listed by itself)",
                                        flop_counter.permute_bytes(T, K, H, elem, 8)),
        "sort_hist_kernel": ("permute (histogram launch)", rows * 8),
        "gather_combine_kernel": ("unpermute forward and permute backward (one kernel, averaged)",
                                  flop_counter.unpermute_bytes(T, K, H, elem)),
        "unpermute_grad_kernel": ("unpermute backward", flop_counter.unpermute_grad_bytes(T, K, H, elem)),
        "swiglu_kernel": ("SwiGLU", flop_counter.swiglu_bytes(rows, F, elem)),
        "swiglu_grad_kernel": ("SwiGLU backward", flop_counter.swiglu_bytes(rows, F, elem, True)),
    }


def cmd_in_layer(args):
    """Durations of the HBM-bound kernels inside the layer step from a rocprofv3 --kernel-trace --stats run of bench.py
    (the `*_kernel_stats.csv`), as fractions of the 8 TB/s peak of their algorithmic bytes."""
    from .build import source_hash
    from .workloads import WORKLOADS

    ops = _in_layer_ops(WORKLOADS[args.workload])
    found = {}
    with open(args.stats, newline="") as fh:
        for row in csv.DictReader(fh):
            name = short_name(row["Name"])
            for frag, (label, nbytes) in ops.items():
                if name.startswith(frag + "<") or name == frag:
                    us = float(row["AverageNs"]) / 1e3
                    found[frag] = {"op": label, "calls": int(row["Calls"]), "avg_us": round(us, 2),
                                   "bytes_per_launch": int(nbytes), "gbs": round(nbytes / us / 1e3, 1),
                                   "frac_of_hbm_peak": round(nbytes / us / 1e3 / 8000.0, 4)}
    print(f"{'kernel':30s} {'calls':>6s} {'avg_us':>9s} {'MB':>8s} {'GB/s':>8s} {'of 8 TB/s':>10s}  op")
    for frag, r in found.items():
        print(f"{frag:30s} {r['calls']:6d} {r['avg_us']:9.2f} {r['bytes_per_launch'] / 1e6:8.1f} {r['gbs']:8.1f} "
              f"{r['frac_of_hbm_peak']:10.3f}  {r['op']}")
    if args.out:
        data = {}
        if os.path.exists(args.out):
            with open(args.out) as fh:
                data = json.load(fh)
        build = source_hash()
        if data.get("build") != build:
            data = {"build": build, "what": "rocprofv3 --kernel-trace --stats durations of the HBM-bound kernels inside "
                                            "the layer step (bench.py), algorithmic bytes over the average", "kernels": {}}
        data["kernels"][args.workload] = found
        with open(args.out, "w") as fh:
            json.dump(data, fh, indent=1, sort_keys=True)
            fh.write("\n")
        print(f"\nrecorded for build {build} in {args.out}")


# ---- power / clock ---------------------------------------------------------------------------------------------
def _hwmon_dirs():
    return sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))


def _read(path):
    try:
        with open(path) as fh:
            return fh.read().strip()
    except OSError:
        return None


def sample_board():
    """(watts, shader MHz) of the first GPU, from the amdgpu hwmon and pp_dpm_sclk files; None where unreadable."""
    watts = mhz = None
    for h in _hwmon_dirs():
        for name in ("power1_input", "power1_average"):
            v = _read(os.path.join(h, name))
            if v is not None:
                watts = int(v) / 1e6
                break
        sclk = _read(os.path.join(os.path.dirname(os.path.dirname(h)), "pp_dpm_sclk"))
        if sclk:
            for line in sclk.splitlines():
                if "*" in line:
                    found = re.search(r"(\d+)\s*Mhz", line, re.I)
                    if found:
                        mhz = int(found.group(1))
        if watts is not None:
            break
    return watts, mhz


def cmd_power(args):
    import torch

    from .ops.gmm import gmm_raw

    if not torch.cuda.is_available():
        raise SystemExit("needs a HIP device")
    dev = torch.device("cuda", 0)
    T, H, F, E = 8192, 4096, 14336, 8
    bf = torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(0)
    counts = torch.full((E,), T // E, dtype=torch.int64, device=dev)
    cap = None
    for h in _hwmon_dirs():
        v = _read(os.path.join(h, "power1_cap"))
        if v is not None:
            cap = int(v) / 1e6
    idle = sample_board()
    print(f"Mixtral-shape fc1 products, {T} rows in {E} equal groups, hidden {H}, 2*ffn {2 * F}, bf16; "
          f"{args.seconds:.0f} s of back-to-back launches per line")
    print(f"board power cap {cap} W; idle reading {idle[0]} W at {idle[1]} MHz")
    print(f"{'product':10s} {'operands':8s} {'ms':>8s} {'TFLOP/s':>8s} {'frac':>6s} {'W(avg)':>8s} {'W(max)':>8s} {'MHz(avg)':>9s}")

    def operand(data, *shape):
        if data == "zeros":
            return torch.zeros(*shape, device=dev, dtype=bf)
        if data == "ones":
            return torch.ones(*shape, device=dev, dtype=bf)
        if data == "small":
            return torch.randint(-2, 3, shape, generator=gen, device=dev).to(bf)
        return torch.randn(*shape, generator=gen, device=dev).to(bf)

    flops = 2 * T * H * 2 * F
    for mode in args.modes.split(","):
        for data in args.data.split(","):
            if mode == "fwd1":
                x, w = operand(data, T, H), operand(data, E, H, 2 * F)
                fn = lambda: gmm_raw(x, w, counts, 0, 1)            # noqa: E731
            elif mode == "dx1":
                dy, w = operand(data, T, 2 * F), operand(data, E, H, 2 * F)
                fn = lambda: gmm_raw(dy, w.transpose(1, 2), counts, 0, 1)   # noqa: E731
            elif mode == "dw1":
                x, dy = operand(data, T, H), operand(data, T, 2 * F)
                fn = lambda: gmm_raw(x.t(), dy, counts, 2, 1)      # noqa: E731
            elif mode == "library":   # torch.bmm (the vendor library) on the same shape as E dense products, for orientation
                x, w = operand(data, E, T // E, H), operand(data, E, H, 2 * F)
                fn = lambda: torch.bmm(x, w)                       # noqa: E731
            else:
                raise SystemExit(f"unknown mode {mode}")
            for _ in range(30):
                fn()
            torch.cuda.synchronize()
            samples = []
            stop = threading.Event()

            def sampler():
                while not stop.is_set():
                    samples.append(sample_board())
                    time.sleep(0.2)
            thread = threading.Thread(target=sampler)
            thread.start()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0, n = time.time(), 0
            e0.record()
            while time.time() - t0 < args.seconds:
                for _ in range(50):
                    fn()
                torch.cuda.synchronize()
                n += 50
            e1.record()
            torch.cuda.synchronize()
            stop.set()
            thread.join()
            ms = e0.elapsed_time(e1) / n
            steady = samples[len(samples) // 4:] or samples       # drop the ramp at the start
            watts = [s[0] for s in steady if s[0] is not None]
            mhz = [s[1] for s in steady if s[1] is not None]
            tf = flops / ms / 1e9
            print(f"{mode:10s} {data:8s} {ms:8.4f} {tf:8.0f} {tf / 2500:6.3f} "
                  f"{(sum(watts) / len(watts)) if watts else float('nan'):8.0f} {max(watts) if watts else float('nan'):8.0f} "
                  f"{(sum(mhz) / len(mhz)) if mhz else float('nan'):9.0f}", flush=True)
            del fn
            time.sleep(1.0)


def _products(dev, data, gen, counts=None):
    """fc1-shaped products of the Mixtral expert MLP: name -> (callable, flops).  counts: rows per expert (eight equal
    groups by default)."""
    import torch

    from .ops.gmm import gmm_raw

    T, H, F, E = 8192, 4096, 14336, 8
    bf = torch.bfloat16
    if counts:
        T, E = sum(counts), len(counts)
        counts = torch.tensor(counts, dtype=torch.int64, device=dev)
    else:
        counts = torch.full((E,), T // E, dtype=torch.int64, device=dev)

    def operand(*shape):
        if data == "zeros":
            return torch.zeros(*shape, device=dev, dtype=bf)
        return torch.randn(*shape, generator=gen, device=dev).to(bf)

    def make(mode):
        if mode == "fwd1":
            x, w = operand(T, H), operand(E, H, 2 * F)
            return lambda: gmm_raw(x, w, counts, 0, 1)
        if mode == "dx1":
            dy, w = operand(T, 2 * F), operand(E, H, 2 * F)
            return lambda: gmm_raw(dy, w.transpose(1, 2), counts, 0, 1)
        if mode == "dw1":
            x, dy = operand(T, H), operand(T, 2 * F)
            return lambda: gmm_raw(x.t(), dy, counts, 2, 1)
        raise SystemExit(f"unknown mode {mode}")
    return make, 2 * T * H * 2 * F


def cmd_timeline(args):
    import ctypes

    import numpy as np
    import torch

    from . import _lib

    if not torch.cuda.is_available():
        raise SystemExit("needs a HIP device")
    lib = _lib.load()
    if not hasattr(lib, "ms_trace_read"):
        raise SystemExit("this library has no tile trace: build it with `python -m mindspeed_amd.build --trace` and "
                         "select it with MINDSPEED_AMD_LIB=mindspeed_amd/libmindspeed_amd_trace.so")
    lib.ms_trace_read.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.ms_trace_read.restype = ctypes.c_int
    lib.ms_trace_clear.argtypes = []
    lib.ms_trace_clear.restype = ctypes.c_int
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev).manual_seed(0)
    slots = 16384
    counts = [int(c) for c in args.counts.split(",")] if args.counts else None
    groups = f"{sum(counts)} rows in groups of {args.counts}" if counts else "8192 rows in 8 equal groups"
    print(f"Mixtral-shape fc1 products ({groups}, hidden 4096, 2*ffn 28672, bf16), one launch each; "
          "times in microseconds from a 100 MHz clock, averaged over the workgroups that held a tile"
          + (" of the given height (rows)" if counts else ""))
    print(f"{'product':8s} {'operands':8s} {'tiles':>6s} {'find tile':>10s} {'first data':>11s} {'K loop':>9s} {'epilogue':>9s} "
          f"{'tile total':>11s} {'idle gap':>9s} {'launch span':>12s} {'MFMA share':>11s}")
    for data in args.data.split(","):
        make, flops = _products(dev, data, gen, counts)
        for mode in args.modes.split(","):
            fn = make(mode)
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            _lib.check(lib.ms_trace_clear(), "ms_trace_clear")
            fn()
            torch.cuda.synchronize()
            buf = (ctypes.c_longlong * (slots * 8))()
            _lib.check(lib.ms_trace_read(buf, slots * 8), "ms_trace_read")
            rec = np.frombuffer(buf, dtype=np.int64).reshape(-1, 8)
            rec = rec[(rec[:, 0] >> 40) == 1]
            rec = rec[rec[:, 4] > rec[:, 1]]          # workgroups that held a tile
            if len(rec) == 0:
                print(f"{mode:8s} {data:8s} no records")
                continue
            heights = sorted(set(int(h) for h in rec[:, 6]), reverse=True)
            if len(heights) > 1:                       # ragged groups: the phases of each tile height by itself
                for h in heights:
                    sub = rec[rec[:, 6] == h]
                    ush = lambda a, b: float((sub[:, a] - sub[:, b]).mean()) / 100.0     # noqa: E731
                    print(f"{mode + ' ' + str(h):8s} {data:8s} {len(sub):6d} {ush(2, 1):10.2f} {ush(3, 2):11.2f} {ush(4, 3):9.2f} "
                          f"{ush(5, 4):9.2f} {ush(5, 1):11.2f}", flush=True)
            us = lambda a, b: float((rec[:, a] - rec[:, b]).mean()) / 100.0     # noqa: E731
            gaps = []
            by_cu = {}
            for r in rec:
                by_cu.setdefault(int(r[0]) & ((1 << 40) - 1), []).append((int(r[1]), int(r[5])))
            for runs in by_cu.values():
                runs.sort()
                gaps += [b[0] - a[1] for a, b in zip(runs, runs[1:])]
            span = float(rec[:, 5].max() - rec[:, 1].min()) / 100.0
            # MFMA time of a 256 x 256 tile: 2 * 256 * 256 * K flops at 1024 flop / clock / SIMD x 4 SIMDs, 2.4 GHz
            tiles_total = len(rec)
            mfma_us = flops / tiles_total / (4 * 1024 * 2.4e9) * 1e6
            total = us(5, 1)
            print(f"{mode:8s} {data:8s} {tiles_total:6d} {us(2, 1):10.2f} {us(3, 2):11.2f} {us(4, 3):9.2f} {us(5, 4):9.2f} "
                  f"{total:11.2f} {(sum(gaps) / len(gaps) / 100.0) if gaps else float('nan'):9.2f} {span:12.1f} "
                  f"{mfma_us / total:11.3f}", flush=True)
            del fn


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    t = sub.add_parser("traffic")
    t.add_argument("--fetch", required=True)
    t.add_argument("--write", required=True)
    t.add_argument("--workload", default="mixtral")
    t.add_argument("--copy-mib", type=int, default=1024)
    t.add_argument("--out", default="")
    c = sub.add_parser("counters")
    c.add_argument("files", nargs="+")
    c.add_argument("--all", action="store_true", help="every kernel of the library, not only the grouped matmuls")
    pr = sub.add_parser("products")
    pr.add_argument("--csv", required=True, help="the *_counter_collection.csv of the rocprofv3 --pmc run")
    pr.add_argument("--iters", type=int, default=3)
    il = sub.add_parser("in-layer")
    il.add_argument("--stats", required=True, help="the *_kernel_stats.csv of a rocprofv3 --kernel-trace --stats run")
    il.add_argument("--workload", default="mixtral")
    il.add_argument("--out", default="")
    w = sub.add_parser("power")
    w.add_argument("--seconds", type=float, default=4.0)
    w.add_argument("--modes", default="fwd1,dx1,dw1")
    w.add_argument("--data", default="randn,small,zeros")
    tl = sub.add_parser("timeline")
    tl.add_argument("--modes", default="fwd1,dx1,dw1")
    tl.add_argument("--data", default="randn,zeros")
    tl.add_argument("--counts", default="", help="comma-separated rows per expert instead of eight equal groups")
    args = ap.parse_args()
    {"traffic": cmd_traffic, "counters": cmd_counters, "power": cmd_power, "timeline": cmd_timeline,
     "in-layer": cmd_in_layer, "products": cmd_products}[args.cmd](args)


if __name__ == "__main__":
    sys.exit(main())
