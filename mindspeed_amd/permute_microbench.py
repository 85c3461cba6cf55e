"""The permute / unpermute family in isolation: back-to-back launches through the C ABI.

    python -m mindspeed_amd.permute_microbench [--tokens 4096] [--hidden 4096] [--experts 8] [--topk 2]
                                               [--iters 200] [--warmup 20] [--sets N]

Every op is launched ``--iters`` times in a row on resident buffers (no allocation, no Python op wrapper in
the loop: one ctypes call per launch, which is shorter than the kernels at the default size) between two
events on the launch stream, so the average is the kernel's duration plus the gap between launches.  Rates are
the algorithmic bytes of the op (rows read once and written once, plus its index and probability arrays)
over that average, next to the 8 TB/s HBM peak.  The ops:

    permute         ms_moe_token_permute          sort by expert + row scatter (expert count given)
    permute_mask    ms_moe_routing_map_permute    the same from a [tokens, experts] boolean map
    unpermute       ms_moe_token_unpermute        probability-weighted top-k gather
    unpermute_grad  ms_moe_token_unpermute_grad   grad of rows and of probabilities
    permute_grad    ms_moe_token_permute_grad     unweighted top-k gather
    unpermute_mask, unpermute_mask_grad, permute_mask_grad
                    the three gathers above driven by the routing-map form's row map (top-k = experts)
    copy            mb_copy_bytes (helper library) plain copy of the permuted rows, for orientation
"""
from __future__ import annotations

import argparse
import ctypes

import torch

from . import _lib, flop_counter, microbench_kernels

HBM_PEAK_GBS = 8000.0


def measure(num_tokens=4096, hidden=4096, num_experts=8, topk=2, dtype=torch.bfloat16, iters=200, warmup=20,
            device=None, sets=1):
    """Returns ``{op: {"avg_us", "gbs", "bytes_per_launch", "frac_of_hbm_peak"}}`` for the ops listed above.

    ``sets`` > 1 rotates the launches through that many separate sets of buffers (inputs and outputs alike), so
    that a launch finds nothing of its operands in the 256 MB last-level cache once the sets together are several
    times larger than it ("cold" figures); with one set, buffers of this size stay resident in that cache."""
    if not torch.cuda.is_available():
        raise RuntimeError("permute_microbench needs a HIP device")
    dev = torch.device("cuda", 0) if device is None else device
    lib = _lib.load()
    mb = microbench_kernels.load()
    T, H, E, K = num_tokens, hidden, num_experts, topk
    elem = torch.empty(0, dtype=dtype).element_size()
    code = _lib.dtype_code(dtype, "tokens")
    gen = torch.Generator(device=dev).manual_seed(0)
    rows = T * K
    idx = torch.topk(torch.randn(T, E, generator=gen, device=dev), K, dim=-1)[1].contiguous()   # int64, distinct per token
    rmap = torch.zeros(T, E, dtype=torch.bool, device=dev)
    rmap.scatter_(1, idx, True)
    probs = torch.rand(T, K, generator=gen, device=dev).to(dtype)
    probs_mask = torch.zeros(T, E, dtype=dtype, device=dev).scatter_(1, idx, probs)
    nbytes = ctypes.c_size_t(0)
    _lib.check(lib.ms_moe_token_permute_workspace_size(T, K, E, ctypes.byref(nbytes)), "workspace_size")
    ws_bytes = nbytes.value
    _lib.check(lib.ms_moe_routing_map_workspace_size(T, E, 0, ctypes.byref(nbytes)), "workspace_size")
    ws_mask_bytes = nbytes.value

    class Set:
        """One set of buffers: every large array an op reads or writes."""
        def __init__(self):
            self.x = torch.randn(T, H, generator=gen, device=dev).to(dtype)
            self.gy = torch.randn(T, H, generator=gen, device=dev).to(dtype)
            self.perm = torch.empty(rows, H, dtype=dtype, device=dev)
            self.out = torch.empty(T, H, dtype=dtype, device=dev)
            self.gperm = torch.empty_like(self.perm)
            self.copy_dst = torch.empty_like(self.perm)
            self.row_id_map = torch.empty(rows, dtype=torch.int32, device=dev)
            self.sorted_idx = torch.empty(rows, dtype=torch.int32, device=dev)
            self.counts = torch.empty(E, dtype=torch.int64, device=dev)
            self.mask_map = torch.empty(T * E, dtype=torch.int32, device=dev)
            self.mask_sorted = torch.empty(rows, dtype=torch.int32, device=dev)
            self.gprobs = torch.empty_like(probs)
            self.gprobs_mask = torch.empty_like(probs_mask)
            self.ws = _lib.workspace(ws_bytes, dev)
            self.ws_mask = _lib.workspace(ws_mask_bytes, dev)

    bufs = [Set() for _ in range(max(1, int(sets)))]
    stream = _lib.stream_ptr(dev)
    P = _lib.ptr

    ops = {
        "permute": (lambda b: lib.ms_moe_token_permute(
            stream, P(b.x), P(idx), _lib.MS_INT64, T, K, H, code, rows, E, P(b.perm), P(b.row_id_map), P(b.sorted_idx),
            P(b.counts), P(b.ws), b.ws.numel()), flop_counter.permute_bytes(T, K, H, elem, 8)),
        "permute_mask": (lambda b: lib.ms_moe_routing_map_permute(
            stream, P(b.x), P(rmap), T, E, H, code, rows, 0, P(b.perm), P(b.mask_map), P(b.mask_sorted), P(b.counts),
            P(b.ws_mask), b.ws_mask.numel()), T * H * elem + rows * H * elem + T * E * (1 + 4) + rows * 4),
        "unpermute": (lambda b: lib.ms_moe_token_unpermute(
            stream, P(b.perm), P(b.row_id_map), P(probs), code, T, K, H, code, rows, P(b.out)),
            flop_counter.unpermute_bytes(T, K, H, elem)),
        "unpermute_grad": (lambda b: lib.ms_moe_token_unpermute_grad(
            stream, P(b.perm), P(b.gy), P(b.row_id_map), P(probs), code, T, K, H, code, rows, P(b.gperm), P(b.gprobs)),
            flop_counter.unpermute_grad_bytes(T, K, H, elem)),
        "permute_grad": (lambda b: lib.ms_moe_token_permute_grad(
            stream, P(b.perm), P(b.row_id_map), T, K, H, code, rows, P(b.out)),
            flop_counter.permute_grad_bytes(T, K, H, elem)),
        # the routing-map form of the three gathers: the same entry points with top-k = experts, a [tokens, experts]
        # row map whose unset entries hold an id past the last row, and [tokens, experts] probabilities
        "unpermute_mask": (lambda b: lib.ms_moe_token_unpermute(
            stream, P(b.perm), P(b.mask_map), P(probs_mask), code, T, E, H, code, rows, P(b.out)),
            flop_counter.unpermute_bytes(T, K, H, elem) + T * (E - K) * (4 + elem)),
        "unpermute_mask_grad": (lambda b: lib.ms_moe_token_unpermute_grad(
            stream, P(b.perm), P(b.gy), P(b.mask_map), P(probs_mask), code, T, E, H, code, rows, P(b.gperm),
            P(b.gprobs_mask)), flop_counter.unpermute_grad_bytes(T, K, H, elem) + T * (E - K) * (4 + 2 * elem)),
        "permute_mask_grad": (lambda b: lib.ms_moe_token_permute_grad(
            stream, P(b.perm), P(b.mask_map), T, E, H, code, rows, P(b.out)),
            flop_counter.permute_grad_bytes(T, K, H, elem) + T * (E - K) * 4),
        "copy": (lambda b: mb.mb_copy_bytes(stream, P(b.perm), P(b.copy_dst), b.perm.numel() * elem),
                 2 * rows * H * elem),
    }
    result = {}
    n = len(bufs)
    with torch.cuda.device(dev):
        for name, (launch, work) in ops.items():   # "permute" runs first: the later ops read its outputs
            for i in range(max(warmup, n)):        # every set is touched at least once
                _lib.check(launch(bufs[i % n]), name)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(iters):
                launch(bufs[i % n])
            e1.record()
            torch.cuda.synchronize(dev)
            us = e0.elapsed_time(e1) * 1e3 / iters
            gbs = work / us / 1e3
            result[name] = {"avg_us": round(us, 2), "gbs": round(gbs, 1), "bytes_per_launch": int(work),
                            "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
    return result


def sets_for_cold(num_tokens, hidden, topk, elem=2, footprint=1536 << 20):
    """Number of buffer sets whose large arrays together exceed ``footprint`` bytes (six times the 256 MB cache)."""
    per_set = (3 * num_tokens + 3 * num_tokens * topk) * hidden * elem
    return max(2, -(-footprint // per_set))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--tokens", type=int, default=4096)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--experts", type=int, default=8)
    ap.add_argument("--topk", type=int, default=2)
    ap.add_argument("--iters", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sets", type=int, default=1,
                    help="rotate through this many buffer sets (0: as many as exceed the last-level cache six times)")
    a = ap.parse_args()
    sets = a.sets if a.sets > 0 else sets_for_cold(a.tokens, a.hidden, a.topk)
    res = measure(a.tokens, a.hidden, a.experts, a.topk, torch.bfloat16, a.iters, a.warmup, sets=sets)
    print(f"{a.tokens} tokens x hidden {a.hidden}, {a.experts} experts, top-{a.topk}, bf16; {a.iters} launches per op, "
          f"{sets} buffer set(s)")
    copy = res["copy"]["gbs"]
    for name, r in res.items():
        print(f"{name:19s} {r['avg_us']:8.2f} us  {r['gbs']:8.1f} GB/s  {r['frac_of_hbm_peak']:.3f} of 8 TB/s  "
              f"{r['gbs'] / copy:.2f} of the copy  ({r['bytes_per_launch'] / 1e6:.1f} MB per launch)", flush=True)


if __name__ == "__main__":
    main()
