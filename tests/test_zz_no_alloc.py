"""The grouped-matmul entry point that allocates nothing (ms_gmm_noalloc) against ms_gmm, through the C ABI:
bit-equal outputs on two calls in a row, the second on a smaller problem, so that whatever the first call
left in the library's fixed tile-table buffer must not show in the second."""
import ctypes

import pytest
import torch

from mindspeed_amd import _lib

pytestmark = pytest.mark.gpu


def _call(lib, entry, x, w, gl, group_type, out, accumulate, ws=None):
    dev = x.device
    if group_type == 0:
        (m, k), n = x.shape, w.size(2)
        w_strides = (w.stride(0), w.stride(1), w.stride(2))
    else:
        (k, m), n = x.shape, w.size(1)
        w_strides = (0, w.stride(0), w.stride(1))
    out_dtype = _lib.MS_FP32 if out.dtype == torch.float32 else _lib.dtype_code(out.dtype, "out")
    args = [_lib.stream_ptr(dev), _lib.ptr(x), x.stride(0), x.stride(1), _lib.ptr(w), *w_strides, _lib.ptr(out), n,
            _lib.ptr(gl), 1, group_type, gl.numel(), m, k, n, _lib.dtype_code(x.dtype, "x"), out_dtype,
            1 if accumulate else 0]
    if ws is not None:
        args += [_lib.ptr(ws), ws.numel()]
    _lib.check(getattr(lib, entry)(*args), entry)


def _workspace(lib, num_groups, m, group_type, dev):
    n = ctypes.c_size_t(0)
    _lib.check(lib.ms_gmm_workspace_size(num_groups, m, group_type, ctypes.byref(n)), "ms_gmm_workspace_size")
    return _lib.workspace(n.value, dev)


def _counts(total, groups, gen):
    cuts = torch.sort(torch.randint(0, total + 1, (groups - 1,), generator=gen))[0]
    c = torch.diff(torch.cat([torch.tensor([0]), cuts, torch.tensor([total])]))
    c[groups // 2] += c[0]          # one empty group in front
    c[0] = 0
    return c.long()


# (M, K, N, groups, dtype): a large problem first, then a smaller one with fewer groups
CASES = [
    [(4096, 512, 768, 300, torch.bfloat16), (1000, 200, 328, 5, torch.bfloat16)],
    [(2048, 256, 512, 64, torch.float16), (37, 19, 23, 3, torch.float32)],
]


@pytest.mark.parametrize("pair", CASES)
def test_noalloc_matches_ms_gmm_on_two_calls_in_a_row(pair, device):
    lib = _lib.load()
    gen = torch.Generator().manual_seed(21)
    for M, K, N, E, dtype in pair:
        print("ms_gmm_noalloc case", M, K, N, E, dtype, flush=True)
        counts = _counts(M, E, gen)
        x = torch.randn(M, K, generator=gen).to(dtype).to(device)
        w = (torch.randn(E, K, N, generator=gen) * 0.05).to(dtype).to(device)
        gy = torch.randn(M, N, generator=gen).to(dtype).to(device)
        gl = counts.to(device)
        # forward (split on rows), dX (weight read transposed), dW (split on the reduction dim), fp32 `+=`
        forms = [
            (x, w, 0, torch.empty(M, N, dtype=dtype, device=device), False),
            (gy, w.transpose(1, 2), 0, torch.empty(M, K, dtype=dtype, device=device), False),
            (x.t(), gy, 2, torch.empty(E, K, N, dtype=dtype, device=device), False),
            (x.t(), gy, 2, torch.randn(E, K, N, generator=gen).to(device), True),
        ]
        for a, b, group_type, out, accumulate in forms:
            ref = out.clone()
            ws = _workspace(lib, E, M, group_type, device)
            _call(lib, "ms_gmm", a, b, gl, group_type, ref, accumulate, ws)
            got = out.clone()
            _call(lib, "ms_gmm_noalloc", a, b, gl, group_type, got, accumulate)
            torch.cuda.synchronize()
            assert torch.equal(got, ref), (M, K, N, E, dtype, group_type, accumulate)


def test_noalloc_rejects_more_groups_than_its_buffer_holds(device):
    lib = _lib.load()
    x = torch.zeros(8, 8, dtype=torch.bfloat16, device=device)
    w = torch.zeros(1025, 8, 8, dtype=torch.bfloat16, device=device)
    gl = torch.zeros(1025, dtype=torch.int64, device=device)
    out = torch.empty(8, 8, dtype=torch.bfloat16, device=device)
    with pytest.raises(_lib.MindSpeedAmdError, match="num_groups"):
        _call(lib, "ms_gmm_noalloc", x, w, gl, 0, out, False)
