"""CPU-side checks of the C ABI: the library loads without a GPU, exports every symbol the header declares, its
host-only quant-parameter functions agree with the oracle, and device entry points fail cleanly (status code, no
crash) when there is no GPU or the arguments are invalid."""
import ctypes as C
import os
import random
import re

import numpy as np
import pytest

from mindspore_amd import lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(lib.LIB_PATH):
        from mindspore_amd import build
        build.build_library()
    return lib.load()


def test_exports_match_header(L):
    header = open(os.path.join(ROOT, "include", "mi355x_int8.h")).read()
    declared = set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", header))
    assert declared == set(lib.EXPORTS), declared ^ set(lib.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert b"gfx950" in L.mi_version()


def test_measurement_aids_live_in_their_own_library(L):
    """The benchmark's probes are declared in include/mi355x_diag.h and built into libmi355x_diag.so: the header an
    integrator reads and the product library carry none of them."""
    header = open(os.path.join(ROOT, "include", "mi355x_diag.h")).read()
    declared = set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", header))
    assert declared == set(lib.DIAG_EXPORTS), declared ^ set(lib.DIAG_EXPORTS)
    D = lib.load_diag()
    for name in declared:
        assert hasattr(D, name) and not hasattr(L, name), name
    assert D.mi_diag_stream_read(None, 16, None) == lib.MI_NULL_PTR
    assert D.mi_diag_copy(None, None, 16, None) == lib.MI_NULL_PTR
    assert D.mi_diag_mfma_rate(None, 1, 1, None, None) == lib.MI_NULL_PTR


def test_quantize_multiplier_matches_oracle(L, orc):
    rnd = random.Random(11)
    vals = [0.0, 1.0, 0.5, 0.9999999999999999, 1e-9, 123.0, -0.3, 5e-324, float("inf"), float("nan")]
    vals += [rnd.uniform(1e-7, 3.0) for _ in range(5000)]
    for m in vals:
        mult, ls, rs = C.c_int32(), C.c_int32(), C.c_int32()
        assert L.mi_quantize_multiplier(m, C.byref(mult), C.byref(ls), C.byref(rs)) == 0
        assert (mult.value, ls.value, rs.value) == orc.round_param(m), m


def test_quantize_multiplier_single_matches_oracle(L, orc):
    rnd = random.Random(12)
    vals = [0.0, 0.5, 1.0, 8388608.0, 8388613.0, 4294967295.0] + [rnd.uniform(0, 2.0 ** 32 - 1) for _ in range(2000)]
    vals += [rnd.uniform(0, 3.0) for _ in range(500)]
    for m in vals:
        mult, ls, rs = C.c_int32(), C.c_int32(), C.c_int32()
        assert L.mi_quantize_multiplier_single(m, C.byref(mult), C.byref(ls), C.byref(rs)) == 0
        assert (mult.value, ls.value, rs.value) == orc.round_param_single(m), m
    for bad in (-1.0, 2.0 ** 32, float("nan")):
        assert L.mi_quantize_multiplier_single(bad, C.byref(mult), C.byref(ls), C.byref(rs)) == -3


def test_requant_params_and_act_range_match_oracle(L, orc):
    rng = np.random.default_rng(12)
    sw = rng.uniform(1e-4, 1e-2, 1000)
    for sx, so in [(0.02, 0.05), (0.7, 1e-5), (0.0123, 0.4)]:
        mult, ls, rs = (np.empty(1000, np.int32) for _ in range(3))
        p = lambda a, t=C.c_int32: a.ctypes.data_as(C.POINTER(t))
        assert L.mi_requant_params(sx, p(sw, C.c_double), 1000, so, p(mult), p(ls), p(rs)) == 0
        m2, l2, r2 = orc.requant_params(sx, sw, so)
        assert np.array_equal(mult, m2) and np.array_equal(ls, l2) and np.array_equal(rs, r2)
    for _ in range(2000):
        zp, scale = int(rng.integers(-128, 128)), float(np.float32(rng.uniform(1e-3, 0.5)))
        for act, (relu, relu6) in [(0, (0, 0)), (1, (1, 0)), (3, (0, 1))]:
            lo, hi = C.c_int32(), C.c_int32()
            assert L.mi_activation_range(act, zp, scale, C.byref(lo), C.byref(hi)) == 0
            assert (lo.value, hi.value) == orc.act_range(relu, relu6, zp, scale)


def test_multiply_by_quantized_multiplier_matches_oracle(L, orc):
    rnd = random.Random(13)
    for _ in range(20000):
        v = rnd.randint(-2 ** 31, 2 ** 31 - 1)
        mult = rnd.randint(1 << 30, 2 ** 31 - 1) * rnd.choice([1, 1, -1])
        ls, rs = (0, -rnd.randint(0, 31)) if rnd.random() < 0.7 else (rnd.randint(0, 8), 0)
        assert L.mi_multiply_by_quantized_multiplier(v, mult, ls, rs) == orc.mul_by_quant_mult(v, mult, ls, rs)
    assert L.mi_multiply_by_quantized_multiplier(-2 ** 31, -2 ** 31, 0, 0) == 2 ** 31 - 1


def test_same_pad(L):
    # the stem of the MobileNet block: 224 -> 112, kernel 3, stride 2: pad (0, 1)
    b, a, o = C.c_int32(), C.c_int32(), C.c_int32()
    assert L.mi_conv_same_pad(224, 3, 2, 1, C.byref(b), C.byref(a), C.byref(o)) == 0
    assert (b.value, a.value, o.value) == (0, 1, 112)
    assert L.mi_conv_same_pad(112, 3, 1, 1, C.byref(b), C.byref(a), C.byref(o)) == 0
    assert (b.value, a.value, o.value) == (1, 1, 112)
    assert L.mi_conv_same_pad(5, 1, 2, 1, C.byref(b), C.byref(a), C.byref(o)) == 0
    assert (b.value, a.value, o.value) == (0, 0, 3)
    assert L.mi_conv_same_pad(0, 3, 1, 1, C.byref(b), C.byref(a), C.byref(o)) == lib.MI_PARAM_INVALID


def test_device_entry_points_fail_cleanly_without_init(L):
    """No GPU work is launched for invalid calls: null handles / pointers give MI_NULL_PTR; creating a kernel before
    a successful mi_init gives a status, never a crash."""
    assert L.mi_matmul_run(None, None, 4, None, None) == lib.MI_NULL_PTR
    assert L.mi_conv_run(None, None, 1, 4, 4, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynmm_run(None, None, 1, 0.1, 0, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynquant_run(None, None, 4, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynquant_run_segments(None, None, 4, 4, None, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynquant_run_segments_host(None, None, 4, 4, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynmm_run_rows(None, None, 1, None, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynmm_run_rows_host(None, None, 1, None, 0, None) == lib.MI_NULL_PTR
    assert L.mi_device_malloc(64, None) == lib.MI_NULL_PTR
    assert L.mi_copy_to_device(None, None, 8, None) == lib.MI_NULL_PTR
    assert L.mi_copy_to_host(None, None, 8, None) == lib.MI_NULL_PTR
    assert L.mi_copy_to_device(None, None, 0, None) == lib.MI_OK and L.mi_device_free(None) == lib.MI_OK
    h = C.c_void_p()
    assert L.mi_matmul_create(None, None, None, C.byref(h)) == lib.MI_NULL_PTR
    import torch
    if not torch.cuda.is_available():
        scales = (C.c_double * 1)(0.1)
        zps = (C.c_int32 * 1)(0)
        d = lib.MatmulDesc(8, 4, 1, 0, 0.1, 0, 0.1, 0, 1, scales, zps)
        w = np.zeros((4, 8), np.int8)
        rc = L.mi_matmul_create(C.byref(d), w.ctypes.data, None, C.byref(h))
        assert rc == lib.MI_ERROR and b"mi_init" in L.mi_last_error()
        p = C.c_void_p()
        assert L.mi_device_malloc(64, C.byref(p)) == lib.MI_ERROR and p.value is None
        assert L.mi_stream_synchronize(None) == lib.MI_ERROR
        d3 = lib.ConvDesc(4, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0.1, 0, 0.1, 0, 1, scales, zps, 2)
        assert L.mi_conv_create(C.byref(d3), np.zeros((8, 3, 3, 4), np.int8).ctypes.data, None,
                                C.byref(h)) == lib.MI_PARAM_INVALID  # unknown flag bit
        assert L.mi_init(0) == lib.MI_NOT_SUPPORT


def test_public_header_is_plain_c(tmp_path):
    """include/mi355x_int8.h is the drop-in boundary: it has to compile as C99 and as C++11 on its own."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "mi355x_int8.h"\n'
                   "int main(void) { mi_conv_desc d = {0}; mi_matmul_desc m = {0}; return d.flags + m.deep; }\n")
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    for cmd in (["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror"],
                ["g++", "-std=c++11", "-Wall", "-Werror", "-x", "c++"]):
        p = subprocess.run(cmd + ["-I", inc, "-fsyntax-only", str(src)], capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
