"""Algorithmic work accounting (and optional event timing) per op call.

The reference counts grouped-matmul FLOPs inside its op shims
(``FLOP_COUNT(FlopCounter::gmm_flop_*)``, mindspeed/ops/csrc/cann/gmm.cpp:112-114,
formula in mindspeed/ops/csrc/flop_counter/flop_counter.cpp:286-363:
``sum_g 2 * rows_g * K * N = 2*M*K*N``).  This module keeps the same formula and adds
the algorithmic HBM bytes of the bandwidth-bound ops.  When a ``Recorder`` is
active every op call is bracketed by two events on the stream it launches on,
so per-kernel durations can be read after a synchronise.
"""
from __future__ import annotations

import contextlib
from collections import OrderedDict

import torch

_active = None


def gmm_flops(m, k, n):
    """2*M*K*N for forward, dX and dW alike (flop_counter.cpp:297-303,346-363)."""
    return 2 * int(m) * int(k) * int(n)


def permute_bytes(num_tokens, topk, hidden, elem, idx_bytes, num_out=None):
    rows = num_tokens * topk if num_out is None else num_out
    return num_tokens * hidden * elem + rows * hidden * elem + num_tokens * topk * idx_bytes + 2 * num_tokens * topk * 4


def unpermute_bytes(num_tokens, topk, hidden, elem, rows=None):
    rows = num_tokens * topk if rows is None else rows
    return rows * hidden * elem + num_tokens * topk * elem + num_tokens * topk * 4 + num_tokens * hidden * elem


def unpermute_grad_bytes(num_tokens, topk, hidden, elem, rows=None, with_probs=True):
    rows = num_tokens * topk if rows is None else rows
    total = num_tokens * hidden * elem + rows * hidden * elem + num_tokens * topk * 4
    if with_probs:
        total += rows * hidden * elem + 2 * num_tokens * topk * elem
    return total


def permute_grad_bytes(num_tokens, topk, hidden, elem, rows=None):
    rows = num_tokens * topk if rows is None else rows
    return rows * hidden * elem + num_tokens * hidden * elem + num_tokens * topk * 4


def swiglu_bytes(rows, ffn, elem, backward=False):
    """Forward: read gate and up, write the product (3 arrays of rows x ffn).  Backward: read gate, up and the
    incoming gradient, write both halves of the input gradient (5)."""
    return rows * ffn * elem * (5 if backward else 3)


class Recorder:
    """Collects (name, work, unit, start event, end event) for every op call while active."""

    def __init__(self, timing=True):
        self.timing = timing
        self.calls = []

    def summary(self):
        """name -> dict(calls, work, unit, ms) ; call after torch.cuda.synchronize()."""
        out = OrderedDict()
        for name, work, unit, e0, e1 in self.calls:
            s = out.setdefault(name, {"calls": 0, "work": 0, "unit": unit, "ms": 0.0})
            s["calls"] += 1
            s["work"] += work
            if e0 is not None:
                s["ms"] += e0.elapsed_time(e1)
        return out


@contextlib.contextmanager
def record(timing=True):
    global _active
    prev, rec = _active, Recorder(timing)
    _active = rec
    try:
        yield rec
    finally:
        _active = prev


def timing_active() -> bool:
    """True while a recorder is bracketing every op with events (ops then keep to one stream, so that the
    per-op durations are those of kernels running alone)."""
    return _active is not None and _active.timing


class _NoOp:
    __slots__ = ()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NOOP = _NoOp()


class _Bracket:
    __slots__ = ("rec", "name", "work", "unit", "device", "stream", "e0")

    def __init__(self, rec, name, work, unit, device):
        self.rec, self.name, self.work, self.unit, self.device = rec, name, work, unit, device

    def __enter__(self):
        self.e0 = None
        if self.rec.timing:
            self.stream = torch.cuda.current_stream(self.device)
            self.e0 = torch.cuda.Event(enable_timing=True)
            self.e0.record(self.stream)
        return self

    def __exit__(self, exc_type, exc, tb):
        e1 = None
        if self.rec.timing:
            e1 = torch.cuda.Event(enable_timing=True)
            e1.record(self.stream)
        if exc_type is None:
            self.rec.calls.append((self.name, self.work() if callable(self.work) else self.work, self.unit, self.e0, e1))
        return False


def op(name, work, unit, device):
    """Used by the ops around each C-ABI call: ``with op(...):``.  Free when no Recorder is active (``work`` may be a
    callable, evaluated only when one is)."""
    rec = _active
    if rec is None:
        return _NOOP
    return _Bracket(rec, name, work, unit, device)
