"""Measurement helpers that are not part of the product library: ``copy_bytes``, a plain device copy kernel used as
the reference point of the HBM-bound microbenchmarks and to calibrate profiler byte counters.  Lives in
``libmindspeed_amd_microbench.so`` (``python -m mindspeed_amd.build --microbench``; ``__graft_entry__.build()`` builds
it too)."""
from __future__ import annotations

import ctypes
import os

import torch

from . import build as _build

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(_build.MICROBENCH_LIB_PATH):
            raise RuntimeError(f"{_build.MICROBENCH_LIB_PATH} is missing: build it with "
                               "`python -m mindspeed_amd.build --microbench` (needs hipcc)")
        lib = ctypes.CDLL(_build.MICROBENCH_LIB_PATH)
        lib.mb_copy_bytes.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        lib.mb_copy_bytes.restype = ctypes.c_int
        _lib = lib
    return _lib


def copy_bytes(src: torch.Tensor, dst: torch.Tensor, nbytes: int | None = None):
    """``dst[:nbytes] = src[:nbytes]`` (bytes) on the current stream of ``src``'s device."""
    if src.device.type != "cuda" or dst.device != src.device:
        raise RuntimeError("copy_bytes needs two tensors on one HIP device")
    n = src.numel() * src.element_size() if nbytes is None else int(nbytes)
    if n > dst.numel() * dst.element_size() or n > src.numel() * src.element_size():
        raise ValueError("copy_bytes: more bytes than the tensors hold")
    stream = ctypes.c_void_p(torch.cuda.current_stream(src.device).cuda_stream)
    rc = load().mb_copy_bytes(stream, ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), n)
    if rc != 0:
        raise RuntimeError(f"mb_copy_bytes failed with status {rc}")
