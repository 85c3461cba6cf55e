"""ctypes loader for the C counting-sort oracle.  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libpermute_index_oracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.ms_oracle_permute_index.restype = ctypes.c_int
        _lib.ms_oracle_permute_rows.restype = ctypes.c_int
    return _lib


def permute_index(flat, num_experts):
    """Return (forward[int32], inverse[int32], counts[int64]) for flat ids."""
    lib = _load()
    flat = np.ascontiguousarray(flat, dtype=np.int64)
    n = flat.size
    fwd = np.empty(n, dtype=np.int32)
    inv = np.empty(n, dtype=np.int32)
    counts = np.zeros(num_experts, dtype=np.int64)
    rc = lib.ms_oracle_permute_index(
        flat.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(n), ctypes.c_int64(num_experts),
        fwd.ctypes.data_as(ctypes.c_void_p), inv.ctypes.data_as(ctypes.c_void_p),
        counts.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise ValueError(f"ms_oracle_permute_index failed with code {rc}")
    return fwd, inv, counts


def permute_rows(tokens_bytes, forward, num_out, topk):
    """tokens_bytes: uint8 array [T, row_bytes]; returns uint8 [num_out, row_bytes]."""
    lib = _load()
    tokens_bytes = np.ascontiguousarray(tokens_bytes, dtype=np.uint8)
    forward = np.ascontiguousarray(forward, dtype=np.int32)
    row_bytes = tokens_bytes.shape[1]
    out = np.empty((num_out, row_bytes), dtype=np.uint8)
    rc = lib.ms_oracle_permute_rows(
        tokens_bytes.ctypes.data_as(ctypes.c_void_p), forward.ctypes.data_as(ctypes.c_void_p),
        ctypes.c_int64(num_out), ctypes.c_int64(topk), ctypes.c_int64(row_bytes),
        out.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise ValueError(f"ms_oracle_permute_rows failed with code {rc}")
    return out
