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
    assert lib.ms_version() == _lib.ABI_VERSION


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
    # the second query adds room for partial sums only where tail tiles may be split: split on rows, 16-bit output,
    # few rounds of tiles over a long reduction
    base, m2 = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert lib.ms_gmm_workspace_size(8, 8192, 0, ctypes.byref(base)) == 0
    BF16, FP32 = 0, 2
    assert lib.ms_gmm_workspace_size_split(8, 8192, 14336, 4096, 0, BF16, BF16, 0, ctypes.byref(m2)) == 0
    assert base.value + (16 << 20) <= m2.value <= base.value + (32 << 20) + 4096       # fc2 forward of the Mixtral shape
    for args in [(8, 8192, 4096, 28672, 0, BF16, BF16, 0),      # many rounds of tiles
                 (8, 8192, 2048, 4096, 0, BF16, BF16, 0),       # short reduction
                 (8, 8192, 14336, 4096, 2, BF16, BF16, 0),      # split on the reduction dim
                 (8, 8192, 14336, 4096, 0, BF16, FP32, 1),      # fp32 accumulate form
                 (8, 8192, 14336, 4096, 0, FP32, FP32, 0),      # fp32 operands
                 (4, 600, 8192, 512, 0, BF16, BF16, 0)]:        # far less than a round of tiles
        assert lib.ms_gmm_workspace_size_split(*args, ctypes.byref(m2)) == 0
        assert lib.ms_gmm_workspace_size(args[0], args[1], args[4], ctypes.byref(base)) == 0
        assert m2.value == base.value, args
    assert lib.ms_gmm_workspace_size_split(0, 8192, 14336, 4096, 0, BF16, BF16, 0, ctypes.byref(m2)) != 0
    # bad arguments are rejected before anything is launched
    rc = lib.ms_gmm(None, None, 1, 1, None, 1, 1, 1, None, 1, None, 0, 1, 8, 16, 16, 16, 0, 0, 0, None, 0)
    assert rc != 0 and b"group_type" in lib.ms_last_error()
    rc = lib.ms_gmm(None, None, 1, 1, None, 1, 1, 1, None, 1, None, 0, 0, 8, 16, 16, 16, 7, 7, 0, None, 0)
    assert rc != 0 and b"dtype" in lib.ms_last_error()
    rc = lib.ms_swiglu(None, None, None, 0, -1, 16, 0, None)
    assert rc != 0
    rc = lib.ms_moe_token_unpermute(None, None, None, None, 0, 4, 0, 16, 0, 8, None)
    assert rc != 0 and b"topk" in lib.ms_last_error()
    with pytest.raises(_lib.MindSpeedAmdError):
        _lib.check(rc, "ms_moe_token_unpermute")


def test_tile_order_visits_every_tile_once():
    """The order in which the grouped-matmul kernels walk the tiles of a group (blocks of 4 row tiles x 8 column
    panels, partly filled blocks at both edges, a single left-over row tile joining the last block) is a bijection
    for every group shape up to 40 x 40, and where the sides are multiples of 4 and 8 every run of 32 consecutive
    indices is one 4 x 8 block."""
    lib = _lib.load()
    row, col = ctypes.c_int(-1), ctypes.c_int(-1)
    for R in range(1, 41):
        for C in range(1, 41):
            seen = set()
            order = []
            for i in range(R * C):
                assert lib.ms_gmm_tile_order(R, C, i, ctypes.byref(row), ctypes.byref(col)) == 0
                assert 0 <= row.value < R and 0 <= col.value < C, (R, C, i, row.value, col.value)
                seen.add((row.value, col.value))
                order.append((row.value, col.value))
            assert len(seen) == R * C, (R, C)
            if R % 4 == 0 and C % 8 == 0:
                for b in range(0, R * C, 32):
                    chunk = order[b:b + 32]
                    assert len({r for r, _ in chunk}) == 4 and len({c for _, c in chunk}) == 8, (R, C, b)
    assert lib.ms_gmm_tile_order(4, 4, 16, ctypes.byref(row), ctypes.byref(col)) != 0
    assert lib.ms_gmm_tile_order(0, 4, 0, ctypes.byref(row), ctypes.byref(col)) != 0


def test_launch_has_slots_for_every_table_the_schedule_can_write():
    """Workgroups per XCD of a grouped-matmul launch against the most slots a tile table can need (host arithmetic).
    Common table: every group's eighth of its tiles, rounded up.  Per-XCD lists with the split on the reduction dim:
    the XCD with the most groups holds ceil(G / 8) output blocks, e.g. 3 of 17, which is more than an eighth of all
    tiles when G is not a multiple of 8."""
    lib = _lib.load()
    slots = ctypes.c_int64(0)
    cdiv = lambda a, b: -(-a // b)
    for G in (1, 8, 16, 17, 20, 23, 24, 31, 33, 64, 100, 255, 256):
        for k, n in ((2048, 8192), (2880, 2880), (256, 256), (4096, 4096), (8, 8), (1000, 520)):
            out_tiles = cdiv(k, 256) * cdiv(n, 256)
            for lists in (0, 1):
                assert lib.ms_gmm_launch_slots(G, 4096, k, n, 2, lists, 0, ctypes.byref(slots)) == 0
                need_common = G * cdiv(out_tiles, 8)
                assert slots.value >= need_common, (G, k, n, lists, slots.value, need_common)
                if lists:
                    need_lists = cdiv(G, 8) * out_tiles
                    assert slots.value >= need_lists, (G, k, n, slots.value, need_lists)
    # split on rows: at most ceil(m / 256) + G + 1 row tiles (every group and the zero-fill pseudo-group may end in a
    # partly filled one); with lists the fullest XCD holds at most 1.03 times an eighth of the groups' tiles plus its
    # eighth of the pseudo-group's, rounded up
    for G in (8, 17, 64, 256):
        for m, n in ((8192, 4096), (65536, 2816), (100, 8)):
            tiles = (cdiv(m, 256) + G + 1) * cdiv(n, 256)
            assert lib.ms_gmm_launch_slots(G, m, 4096, n, 0, 1, 0, ctypes.byref(slots)) == 0
            assert slots.value >= cdiv(tiles * 103, 800) + 1
            assert lib.ms_gmm_launch_slots(G, m, 4096, n, 0, 0, 1, ctypes.byref(slots)) == 0
            assert slots.value >= cdiv(tiles + 256, 8) + G
    assert lib.ms_gmm_launch_slots(0, 1, 1, 1, 0, 0, 0, ctypes.byref(slots)) != 0
    assert lib.ms_gmm_launch_slots(8, 1, 1, 1, 1, 0, 0, ctypes.byref(slots)) != 0
