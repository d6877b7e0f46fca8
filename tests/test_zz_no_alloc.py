"""mi_matmul_run_noalloc (the entry point that allocates nothing) against mi_matmul_run and the CPU oracle, through
the C ABI: two calls in a row on one handle, the second with a smaller input; shapes that use both parts of the
scratch area, one part, or none; the size limit."""
import ctypes as C

import numpy as np
import pytest

from mindspore_amd import kernels as K
from mindspore_amd import lib
from mindspore_amd.kernels import QuantParam as QP

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20


def _case(rng, n, k, zwnz):
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    zw = rng.integers(-10, 11, n).astype(np.int32) if zwnz else np.zeros(n, np.int32)
    bias = rng.integers(-5000, 5001, n).astype(np.int32)
    sx, zx = 0.03, int(rng.integers(-20, 21))
    so, zo = float(sx * sw.mean() * np.sqrt(k) * 100.0), int(rng.integers(-20, 21))
    return dict(w=w, bias=bias, sx=sx, zx=zx, sw=sw, zw=zw, so=so, zo=zo, act=0, b_transpose=True)


def _run(L, fn, kern, a, n, offset_in=0, offset_out=0):
    """Calls fn(handle, a_dev, rows, c_dev, stream) on device buffers whose addresses are `offset` bytes past an
    aligned base, returns the output as a NumPy array."""
    import torch
    rows, k = a.shape
    a_buf = torch.zeros(rows * k + 64, dtype=torch.int8, device="cuda")
    c_buf = torch.full((rows * n + 64,), 77, dtype=torch.int8, device="cuda")
    a_buf[offset_in:offset_in + rows * k] = torch.from_numpy(a.reshape(-1)).cuda()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = fn(kern._h, a_buf.data_ptr() + offset_in, rows, c_buf.data_ptr() + offset_out, stream)
    assert rc == lib.MI_OK, (rc, L.mi_last_error())
    torch.cuda.synchronize()
    out = c_buf.cpu().numpy()
    assert np.all(out[:offset_out] == 77) and np.all(out[offset_out + rows * n:] == 77), "wrote outside the output"
    return out[offset_out:offset_out + rows * n].reshape(rows, n)


@pytest.mark.parametrize("n,k,off_in,off_out", [
    (30, 1000, 0, 0),     # deep % 16 != 0 and col % 4 != 0: padded activation rows and padded output, both in scratch
    (64, 1000, 0, 0),     # padded activation rows only
    (30, 1024, 0, 0),     # padded output only
    (256, 512, 0, 0),     # nothing in scratch
    (256, 512, 5, 3),     # misaligned activation and output addresses: both parts again
])
def test_no_alloc_entry_point_matches_the_allocating_one(orc, n, k, off_in, off_out):
    L = lib.load()
    rng = np.random.default_rng(n * 7 + k + off_in)
    orc.set_threads(16)
    case = _case(rng, n, k, zwnz=bool(n & 2))
    kern = K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]),
                              [QP(float(s), int(z)) for s, z in zip(case["sw"], case["zw"])],
                              QP(case["so"], case["zo"]), True, 0)
    # two calls in a row, the second smaller (and on another kernel: 200 rows take GEMM tiles, 7 the decode kernel,
    # 1 the dot kernel); the scratch area keeps the first call's contents in between
    for rows in (200, 7, 300, 1):
        case["a"] = rng.integers(-128, 128, (rows, k), dtype=np.int8)
        want = orc.matmul_int8(**case)
        got_alloc = _run(L, L.mi_matmul_run, kern, case["a"], n, off_in, off_out)
        got = _run(L, L.mi_matmul_run_noalloc, kern, case["a"], n, off_in, off_out)
        assert np.array_equal(got, got_alloc), (n, k, rows)
        assert np.array_equal(got, want), (n, k, rows)


def test_no_alloc_entry_point_rejects_what_does_not_fit():
    import torch
    L = lib.load()
    rng = np.random.default_rng(1)
    case = _case(rng, 30, 1000, False)
    kern = K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]),
                              [QP(float(s), 0) for s in case["sw"]], QP(case["so"], case["zo"]), True, 0)
    per_row = 1008 + 32   # padded activation row + padded output row
    rows_fit = SCRATCH_BYTES // per_row - 8
    rows_over = SCRATCH_BYTES // per_row + 8
    a = torch.zeros(rows_over * 1000, dtype=torch.int8, device="cuda")
    c = torch.full((rows_over * 30,), 55, dtype=torch.int8, device="cuda")
    assert L.mi_matmul_run_noalloc(kern._h, a.data_ptr(), rows_over, c.data_ptr(), None) == lib.MI_PARAM_INVALID
    assert b"scratch" in L.mi_last_error()
    torch.cuda.synchronize()
    assert bool((c == 55).all()), "a rejected call must not launch anything"
    assert L.mi_matmul_run_noalloc(kern._h, a.data_ptr(), rows_fit, c.data_ptr(), None) == lib.MI_OK
    torch.cuda.synchronize()
    assert L.mi_matmul_run_noalloc(None, a.data_ptr(), 1, c.data_ptr(), None) == lib.MI_NULL_PTR
    assert L.mi_matmul_run_noalloc(kern._h, a.data_ptr(), -1, c.data_ptr(), None) == lib.MI_PARAM_INVALID
    assert L.mi_matmul_run_noalloc(kern._h, a.data_ptr(), 0, c.data_ptr(), None) == lib.MI_OK


def test_no_alloc_entry_point_leaves_free_device_memory_unchanged(orc):
    """Free device memory (hipMemGetInfo) before and after a series of calls on fresh shapes: the entry point takes
    its padded rows and padded output from the static scratch area, so nothing may be allocated, whereas the
    allocating entry point grows the handle's workspaces on the same calls."""
    import torch
    L = lib.load()
    rng = np.random.default_rng(9)
    n, k = 1030, 4000  # deep % 16 != 0 and col % 4 != 0: both workspaces are needed
    case = _case(rng, n, k, True)

    def make():
        return K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]),
                                  [QP(float(s), int(z)) for s, z in zip(case["sw"], case["zw"])],
                                  QP(case["so"], case["zo"]), True, 0)
    kern = make()
    rows_list = (900, 1500, 33, 1600)
    a = torch.from_numpy(rng.integers(-128, 128, (max(rows_list), k), dtype=np.int8)).cuda()
    c = torch.empty((max(rows_list), n), dtype=torch.int8, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for rows in rows_list:
        assert L.mi_matmul_run_noalloc(kern._h, a.data_ptr(), rows, c.data_ptr(), stream) == lib.MI_OK
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    got = c[:rows_list[-1]].cpu().numpy()
    case["a"] = a[:rows_list[-1]].cpu().numpy()
    assert np.array_equal(got, orc.matmul_int8(**case))
    # the same calls through the allocating entry point do take device memory (the check above can see allocations)
    for rows in rows_list:
        assert L.mi_matmul_run(kern._h, a.data_ptr(), rows, c.data_ptr(), stream) == lib.MI_OK
    torch.cuda.synchronize()
    free_alloc, _ = torch.cuda.mem_get_info()
    assert free_alloc < free_before
