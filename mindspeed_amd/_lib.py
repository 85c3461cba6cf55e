"""ctypes binding of libmindspeed_amd.so (the C ABI declared in include/mindspeed_amd.h).

The library is the only compute path: if it is missing, or a tensor is not on
a HIP device, the ops raise.  There is no CPU or eager fallback.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# MINDSPEED_AMD_LIB names another build of the same library (to compare two builds on one machine)
LIB_PATH = os.environ.get("MINDSPEED_AMD_LIB") or os.path.join(_HERE, "libmindspeed_amd.so")

ABI_VERSION = 103                # what ms_version() of a matching build returns (argument lists below)
MS_BF16, MS_FP16, MS_FP32 = 0, 1, 2
MS_INT32, MS_INT64 = 0, 1
MS_MAX_EXPERTS = 1024

_DTYPE_CODE = {torch.bfloat16: MS_BF16, torch.float16: MS_FP16, torch.float32: MS_FP32}
_INDEX_CODE = {torch.int32: MS_INT32, torch.int64: MS_INT64}

_c_void_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_size_t = ctypes.c_size_t

# name -> argtypes; every entry point returns int except ms_last_error.
_SIGNATURES = {
    "ms_version": [],
    "ms_moe_token_permute_workspace_size": [_i64, _i64, _i64, ctypes.POINTER(_size_t)],
    "ms_moe_token_permute": [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _int, _i64, _i64,
                             _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _size_t],
    "ms_moe_token_permute_grad": [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _int, _i64, _c_void_p],
    "ms_moe_token_unpermute": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _int, _i64, _c_void_p],
    "ms_moe_token_unpermute_grad": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _int,
                                    _i64, _c_void_p, _c_void_p],
    "ms_moe_routing_map_workspace_size": [_i64, _i64, _int, ctypes.POINTER(_size_t)],
    "ms_moe_routing_map_permute": [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _int, _i64, _int, _c_void_p,
                                   _c_void_p, _c_void_p, _c_void_p, _c_void_p, _size_t],
    "ms_moe_routing_map_probs": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _int, _c_void_p, _c_void_p],
    "ms_moe_routing_map_probs_grad": [_c_void_p, _c_void_p, _i64, _c_void_p, _int, _i64, _c_void_p],
    "ms_moe_zero_unmapped_rows": [_c_void_p, _c_void_p, _i64, _i64, _int, _c_void_p],
    "ms_gmm_workspace_size": [_i64, _i64, _int, ctypes.POINTER(_size_t)],
    "ms_gmm_tile_order": [_int, _int, _int, ctypes.POINTER(_int), ctypes.POINTER(_int)],
    "ms_gmm_launch_slots": [_i64, _i64, _i64, _i64, _int, _int, _int, ctypes.POINTER(_i64)],
    "ms_gmm_workspace_size_split": [_i64, _i64, _i64, _i64, _int, _int, _int, _int, ctypes.POINTER(_size_t)],
    "ms_gmm": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _i64, _i64, _c_void_p, _i64, _c_void_p, _int, _int,
               _i64, _i64, _i64, _i64, _int, _int, _int, _c_void_p, _size_t],
    "ms_gmm_noalloc": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _i64, _i64, _c_void_p, _i64, _c_void_p, _int,
                       _int, _i64, _i64, _i64, _i64, _int, _int, _int],
    "ms_gmm_swiglu": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _i64, _i64, _c_void_p, _i64, _c_void_p, _i64,
                      _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _int, _c_void_p, _size_t],
    "ms_gmm_swiglu_grad_workspace_size": [_i64, _i64, _i64, ctypes.POINTER(_size_t)],
    "ms_gmm_swiglu_grad": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _i64, _i64, _c_void_p, _i64, _c_void_p, _int,
                           _c_void_p, _i64, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _i64, _int, _c_void_p, _size_t],
    "ms_gmm_weight_list": [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _i64, _c_void_p, _i64, _c_void_p, _int,
                           _i64, _i64, _i64, _i64, _int, _int, _c_void_p, _size_t],
    "ms_swiglu": [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _int, _c_void_p],
    "ms_swiglu_grad": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _int, _c_void_p, _c_void_p],
    "ms_sort_chunks": [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _int, _c_void_p, _int,
                       _c_void_p, _c_void_p, _c_void_p],
    "ms_gather_rows": [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _int, _int, _c_void_p],
    "ms_chunk_sort_map": [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p],
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES) + ("ms_last_error",)

_lib = None
_lock = threading.Lock()


class MindSpeedAmdError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP kernels are the only compute path of mindspeed_amd. "
                "Build them with `python -m mindspeed_amd.build` (needs hipcc).")
        lib = ctypes.CDLL(LIB_PATH)
        lib.ms_version.argtypes, lib.ms_version.restype = [], _int
        if lib.ms_version() != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} reports ABI version {lib.ms_version()}, this package binds version "
                               f"{ABI_VERSION}: rebuild it with `python -m mindspeed_amd.build`")
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _int
        lib.ms_last_error.argtypes = []
        lib.ms_last_error.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().ms_last_error().decode("utf-8", "replace")
        raise MindSpeedAmdError(f"{what} failed (status {rc}): {msg}")


def dtype_code(dtype: torch.dtype, what: str) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"{what} dtype [{dtype}] is invalid, should be bfloat16, float16 or float32") from None


def index_code(dtype: torch.dtype, what: str) -> int:
    try:
        return _INDEX_CODE[dtype]
    except KeyError:
        raise TypeError(f"{what} dtype [{dtype}] is invalid, should be int64 or int32") from None


def require_device(t: torch.Tensor, what: str):
    """The kernels run on a HIP device only (meta tensors pass: they only propagate shapes through the
    dispatcher ops' fake kernels)."""
    if t.device.type not in ("cuda", "meta"):
        raise RuntimeError(
            f"{what} is on {t.device}: mindspeed_amd ops run hand-written HIP kernels and need tensors on an "
            "MI355X (torch device type 'cuda' on ROCm); there is no CPU fallback.")


def ptr(t):
    """Device address of a tensor as a plain int (ctypes converts it to the void* argument), None for no tensor."""
    return None if t is None else t.data_ptr()


_raw_stream = torch._C._cuda_getCurrentRawStream


def stream_ptr(device) -> int:
    """The current stream of ``device`` as the integer handle the C ABI takes (a hipStream_t)."""
    index = device.index
    return _raw_stream(torch.cuda.current_device() if index is None else index)


class _Guard:
    """``with on(device):`` makes ``device`` current for the calls inside; free when it already is."""
    __slots__ = ("index", "prev")

    def __init__(self, device):
        self.index = device.index

    def __enter__(self):
        self.prev = -1
        if self.index is not None:
            cur = torch.cuda.current_device()
            if cur != self.index:
                self.prev = cur
                torch.cuda.set_device(self.index)
        return self

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


on = _Guard


def workspace(nbytes: int, device) -> torch.Tensor:
    """Workspace from torch's caching allocator (256-byte granularity, never empty)."""
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
