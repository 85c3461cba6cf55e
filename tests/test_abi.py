"""The C-ABI library loads and exports every symbol include/*.h declares; pure
host-side argument validation works without a GPU (no compute calls here)."""
import ctypes
import glob
import os
import re

import pytest

from mindspeed_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(ms_[a-z0-9_]+)\s*\(", text))
    return names


def test_header_and_binding_agree():
    assert declared_symbols() == set(_lib.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in sorted(declared_symbols()):
        assert hasattr(lib, name), name
    assert lib.ms_version() >= 100


def test_workspace_size_and_validation_are_host_only():
    lib = _lib.load()
    n = ctypes.c_size_t(123)
    assert lib.ms_moe_token_permute_workspace_size(4096, 2, 8, ctypes.byref(n)) == 0 and n.value == 0
    assert lib.ms_moe_token_permute_workspace_size(8192, 8, 64, ctypes.byref(n)) == 0 and n.value == 64 * 64 * 4
    assert lib.ms_moe_token_permute_workspace_size(8192, 8, 0, ctypes.byref(n)) == 0 and n.value == 64 * 1024 * 4
    assert lib.ms_moe_token_permute_workspace_size(8, 2, 5000, ctypes.byref(n)) != 0
    assert b"exceeds" in lib.ms_last_error()
    assert lib.ms_gmm_workspace_size(8, 8192, 0, ctypes.byref(n)) == 0 and n.value >= 8 * 40
    assert lib.ms_gmm_workspace_size(0, 8192, 0, ctypes.byref(n)) != 0
    # bad arguments are rejected before anything is launched
    rc = lib.ms_gmm(None, None, 1, 1, None, 1, 1, 1, None, 1, None, 0, 1, 8, 16, 16, 16, 0, 0, 0, None, 0)
    assert rc != 0 and b"group_type" in lib.ms_last_error()
    rc = lib.ms_gmm(None, None, 1, 1, None, 1, 1, 1, None, 1, None, 0, 0, 8, 16, 16, 16, 7, 7, 0, None, 0)
    assert rc != 0 and b"dtype" in lib.ms_last_error()
    rc = lib.ms_swiglu(None, None, None, 0, -1, 16, 0, None)
    assert rc != 0
    rc = lib.ms_moe_token_unpermute(None, None, None, None, 4, 0, 16, 0, 8, None)
    assert rc != 0 and b"topk" in lib.ms_last_error()
    with pytest.raises(_lib.MindSpeedAmdError):
        _lib.check(rc, "ms_moe_token_unpermute")
