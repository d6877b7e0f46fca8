"""Shape inference of the C ABI (mi_infer_*) against (1) the vectors of the reference's own unit tests that its current
sources still satisfy, (2) the real nnacl inference functions compiled from the reference tree, over seeded random
shapes that include unknown (-1) and degenerate extents, and (3) textbook output-size formulas."""
import random

import pytest

from mindspore_amd import kernels as K
from mindspore_amd.lib import MiError

INFER_ERR, INFER_INVALID = -500, -501


def _call(fn, *args, **kw):
    try:
        return "ok", fn(*args, **kw)
    except MiError as e:
        assert e.code in (INFER_ERR, INFER_INVALID), e
        return ("invalid" if e.code == INFER_INVALID else "error"), None


# mindspore/lite/test/ut/nnacl/infer/matmul_infer_test.cc:26-88 (tests 0 and 1; tests 2 and 3 of that file expect a
# 4-D activation to be flattened and a mismatching K to pass, which the current matmul_infer.c rejects)
MATMUL_KAT = [
    (([4, 3], [4, 3], None, False, True), [4, 4]),
    (([2, 4, 3], [2, 3, 5], None, False, False), [2, 4, 5]),
]
# mindspore/lite/test/ut/nnacl/infer/full_connection_infer_test.cc:27-118
FC_KAT = [
    (([1, 64, 5, 5], [256, 1600]), [1, 256]),
    (([1, 256], [128, 256]), [1, 128]),
    (([1, 128], [3, 128]), [1, 3]),
]
# mindspore/lite/test/ut/nnacl/infer/conv2d_infer_test.cc:26-527 and depthwise_conv2d_infer_test.cc:26-160
# (in, weight, kernel, stride, dilation, pad_mode, pads u/d/l/r, group) -> out; test 1 of each file sets a 7x7 kernel
# on a 3x3 weight, which the current conv2d_infer.c rejects
CONV_KAT = [
    (([5, 4, 4, 6], [20, 3, 3, 6], (3, 3), (1, 1), (1, 1), 0, (1, 1, 1, 1), 1), [5, 4, 4, 20]),
    (([5, 30, 30, 6], [20, 3, 3, 6], (3, 3), (1, 1), (1, 1), 0, (1, 1, 1, 1), 1), [5, 30, 30, 20]),
    (([5, 30, 30, 6], [20, 3, 3, 6], (3, 3), (2, 2), (1, 1), 0, (1, 1, 1, 1), 1), [5, 15, 15, 20]),
    (([5, 120, 120, 6], [20, 5, 5, 6], (5, 5), (2, 2), (1, 1), 0, (0, 0, 0, 0), 1), [5, 58, 58, 20]),
    (([5, 27, 27, 6], [20, 3, 3, 6], (3, 3), (1, 1), (1, 1), 0, (0, 0, 0, 0), 1), [5, 25, 25, 20]),
    (([5, 88, 88, 6], [20, 1, 1, 6], (1, 1), (1, 1), (1, 1), 0, (0, 0, 0, 0), 1), [5, 88, 88, 20]),
    (([5, 11, 11, 6], [20, 9, 1, 6], (9, 1), (1, 1), (1, 1), 0, (4, 4, 0, 0), 1), [5, 11, 11, 20]),
    (([5, 29, 29, 6], [20, 3, 3, 6], (3, 3), (1, 1), (1, 1), 1, (0, 0, 0, 0), 1), [5, 29, 29, 20]),
    (([5, 14, 14, 6], [20, 1, 1, 6], (1, 1), (1, 1), (1, 1), 0, (0, 0, 0, 0), 1), [5, 14, 14, 20]),
    (([5, 448, 448, 6], [20, 5, 5, 6], (5, 5), (2, 2), (1, 1), 1, (0, 0, 0, 0), 1), [5, 224, 224, 20]),
    (([5, 4, 4, 6], [6, 3, 3, 1], (3, 3), (1, 1), (1, 1), 0, (1, 1, 1, 1), 6), [5, 4, 4, 6]),
    (([5, 30, 30, 6], [6, 3, 3, 1], (3, 3), (1, 1), (1, 1), 0, (1, 1, 1, 1), 6), [5, 30, 30, 6]),
]


def test_reference_unit_test_vectors():
    for args, want in MATMUL_KAT:
        assert K.infer_matmul_shape(*args) == want
    for args, want in FC_KAT:
        assert K.infer_fullconnection_shape(*args) == want
    for args, want in CONV_KAT:
        assert K.infer_conv2d_shape(*args)[0] == want


def test_vectors_dropped_as_stale_are_rejected_by_the_real_nnacl(ref):
    assert ref.infer_matmul([1, 128, 1, 1], [96, 128], None, False, True)[0] == "error"
    assert ref.infer_matmul([1, 1288], [256, 1280], None, False, True)[0] == "error"
    assert ref.infer_conv2d([5, 120, 120, 6], [20, 3, 3, 6], (7, 7), (2, 2), (1, 1), 0, (3, 3, 3, 3), 1)[0] == "error"
    for args, want in MATMUL_KAT:
        assert ref.infer_matmul(*args) == ("ok", want)
    for args, want in CONV_KAT:
        assert ref.infer_conv2d(*args)[:2] == ("ok", want)


def test_textbook_cases():
    # vectors: only a pair of vectors collapses to a scalar; a vector against a matrix is promoted to one row first
    assert K.infer_matmul_shape([7], [7]) == []
    assert K.infer_matmul_shape([7], [7, 5]) == [1, 5]
    assert K.infer_matmul_shape([2, 1, 4, 7], [3, 7, 5]) == [2, 3, 4, 5]          # broadcast of leading extents
    assert K.infer_matmul_shape([128, 768], [768, 768], [768], False, True) == [128, 768]
    assert K.infer_matmul_shape([4096, 768], [2304, 768], [1, 2304], False, True) == [4096, 2304]
    assert _call(K.infer_matmul_shape, [4, 3], [4, 5])[0] == "error"
    assert _call(K.infer_matmul_shape, [4, 3], [3, 5], [6])[0] == "error"
    assert _call(K.infer_matmul_shape, [-1, 3], [3, 5])[0] == "invalid"
    assert _call(K.infer_matmul_shape, [2, 4, 3], [3, 3, 5])[0] == "error"       # 2 and 3 do not broadcast
    assert K.infer_fullconnection_shape([2, 3, 4, 5], [10, 20], [10], use_axis=True, axis=2) == [2, 3, 10]
    assert _call(K.infer_fullconnection_shape, [2, 3, 4, 5], [10, 21], use_axis=True, axis=2)[0] == "error"
    assert _call(K.infer_fullconnection_shape, [2, 8], [4, 8], [5])[0] == "error"
    # configuration 2 of the benchmark: stem 3x3 stride 2 SAME on 224 -> 112 with pads (0, 1, 0, 1)
    shape, pads, kernel, group = K.infer_conv2d_shape([1, 224, 224, 3], [32, 3, 3, 3], (-1, -1), (2, 2), (1, 1), 1)
    assert (shape, pads, kernel, group) == ([1, 112, 112, 32], (0, 1, 0, 1), (3, 3), 1)
    # depthwise with group left to the weight
    shape, pads, kernel, group = K.infer_conv2d_shape([1, 112, 112, 192], [192, 3, 3, 1], (3, 3), (1, 1), (1, 1), 1,
                                                      group=0)
    assert (shape, pads, group) == ([1, 112, 112, 192], (1, 1, 1, 1), 192)
    for n, k, s, d in [(17, 3, 2, 1), (17, 3, 2, 2), (9, 5, 3, 1), (224, 7, 2, 1), (5, 5, 1, 1)]:
        span = (k - 1) * d + 1
        got = K.infer_conv2d_shape([1, n, n, 4], [8, k, k, 4], (k, k), (s, s), (d, d), 2)[0]
        assert got == [1, -(-(n - span + 1) // s), -(-(n - span + 1) // s), 8], (n, k, s, d)    # VALID
        got = K.infer_conv2d_shape([1, n, n, 4], [8, k, k, 4], (k, k), (s, s), (d, d), 1)[0]
        assert got == [1, -(-n // s), -(-n // s), 8]                                              # SAME
        got = K.infer_conv2d_shape([1, n, n, 4], [8, k, k, 4], (k, k), (s, s), (d, d), 0, (1, 2, 0, 1))[0]
        assert got == [1, (n + 3 - span) // s + 1, (n + 1 - span) // s + 1, 8]                    # explicit


def _rand_shape(rnd, rank, pool):
    return [rnd.choice(pool) for _ in range(rank)]


def test_matmul_matches_real_nnacl_on_random_shapes(ref):
    rnd = random.Random(2024)
    pool = [1, 1, 2, 2, 3, 4, 4, 6, 8, 0, -1]
    seen = {"ok": 0, "invalid": 0, "error": 0}
    for it in range(6000):
        a = _rand_shape(rnd, rnd.randint(1, 5), pool)
        b = _rand_shape(rnd, rnd.randint(1, 5), pool)
        ta, tb = rnd.random() < 0.3, rnd.random() < 0.5
        if rnd.random() < 0.7 and len(a) >= 2 and len(b) >= 2:   # make the contraction fit most of the time
            kk = a[-2] if ta else a[-1]
            if tb:
                b[-1] = kk
            else:
                b[-2] = kk
        bias = None
        r = rnd.random()
        if r < 0.2:
            bias = [(b[-2] if tb and len(b) >= 2 else b[-1])]
        elif r < 0.3:
            bias = _rand_shape(rnd, rnd.randint(1, 3), [1, 1, 2, 4, b[-1]])
        want = ref.infer_matmul(a, b, bias, ta, tb)
        got = _call(K.infer_matmul_shape, a, b, bias, ta, tb)
        seen[want[0]] += 1
        assert got[0] == want[0], (a, b, bias, ta, tb, want, got)
        if want[0] == "ok":
            assert got[1] == want[1], (a, b, bias, ta, tb, want, got)
    assert min(seen.values()) > 200, seen


def test_fullconnection_matches_real_nnacl_on_random_shapes(ref):
    rnd = random.Random(7)
    pool = [1, 2, 3, 4, 5, 8, 0, -1]
    seen = {"ok": 0, "invalid": 0, "error": 0}
    for it in range(4000):
        a = _rand_shape(rnd, rnd.randint(1, 5), pool[:-2] if rnd.random() < 0.8 else pool)
        use_axis = rnd.random() < 0.5
        axis = rnd.randint(0, len(a) + 1) if use_axis else 0
        n = rnd.choice([1, 3, 16])
        if rnd.random() < 0.75:
            k = 1
            for d in (a[axis:] if use_axis else a[rnd.randint(0, len(a) - 1):]):
                k *= d
        else:
            k = rnd.choice([1, 2, 4, 6, 0])
        w = [n, k]
        has_bias = rnd.random() < 0.5
        bias = [n if rnd.random() < 0.8 else n + 1] if (has_bias != (rnd.random() < 0.1)) else None
        want = ref.infer_fullconnection(a, w, bias, has_bias, use_axis, axis)
        got = _call(K.infer_fullconnection_shape, a, w, bias, has_bias, use_axis, axis)
        seen[want[0]] += 1
        assert got[0] == want[0], (a, w, bias, has_bias, use_axis, axis, want, got)
        if want[0] == "ok":
            assert got[1] == want[1], (a, w, bias, has_bias, use_axis, axis, want, got)
    assert min(seen.values()) > 100, seen


def test_conv2d_matches_real_nnacl_on_random_shapes(ref):
    rnd = random.Random(99)
    seen = {"ok": 0, "invalid": 0, "error": 0}
    for it in range(8000):
        ic = rnd.choice([1, 3, 4, 8, 16])
        mode = rnd.choice(["dense", "depthwise", "grouped", "odd"])
        oc = rnd.choice([1, 4, 8, 16])
        kh, kw = rnd.choice([1, 2, 3, 5, 7]), rnd.choice([1, 2, 3, 5])
        if mode == "dense":
            w, group = [oc, kh, kw, ic], 1
        elif mode == "depthwise":
            w, group = [ic, kh, kw, 1], rnd.choice([ic, 0])
        elif mode == "grouped":
            g = rnd.choice([2, 4])
            w, group = [oc, kh, kw, max(ic // g, 1)], g
        else:
            w, group = [oc, kh, kw, rnd.choice([0, 1, 2, ic])], rnd.choice([0, 1, 2, 3, ic])
        h, wd = rnd.choice([1, 2, 5, 7, 8, 16, 31, 224]), rnd.choice([1, 3, 6, 9, 17, 112])
        x = [rnd.choice([1, 2, 5]), h, wd, ic]
        if rnd.random() < 0.08:
            x[rnd.randint(0, 3)] = -1
        if rnd.random() < 0.03:
            x = x[:rnd.choice([0, 2, 3])]
        kernel = (kh, kw) if rnd.random() < 0.7 else rnd.choice([(-1, -1), (kh, -1), (kh + 1, kw)])
        stride = (rnd.choice([1, 1, 2, 3]), rnd.choice([1, 2, 4])) if rnd.random() < 0.95 else (0, 1)
        dilation = (rnd.choice([1, 1, 2, 3]), rnd.choice([1, 1, 2]))
        pad_mode = rnd.choice([0, 1, 2])
        pads = tuple(rnd.choice([0, 0, 1, 2, 3]) for _ in range(4))
        want = ref.infer_conv2d(x, w, kernel, stride, dilation, pad_mode, pads, group)
        got = _call(K.infer_conv2d_shape, x, w, kernel, stride, dilation, pad_mode, pads, group)
        if len(x) in (2, 3) and want[0] != "invalid":
            # the library only takes 4-D NHWC activations; the reference reads -1 for the missing extents
            assert got[0] == "error"
            continue
        seen[want[0]] += 1
        assert got[0] == want[0], (x, w, kernel, stride, dilation, pad_mode, pads, group, want, got)
        if want[0] == "ok":
            assert (got[1][0], got[1][1], got[1][2], got[1][3]) == (want[1], want[2], want[3], want[4]), \
                (x, w, kernel, stride, dilation, pad_mode, pads, group, want, got)
    assert min(seen.values()) > 200, seen


def test_null_arguments(L=None):
    from mindspore_amd import lib
    import ctypes as C
    lb = lib.load()
    shp = (C.c_int32 * 2)(2, 2)
    out, n = (C.c_int32 * 8)(), C.c_int32()
    assert lb.mi_infer_matmul(shp, 2, shp, 2, None, 0, 0, 0, None, C.byref(n)) == -2
    assert lb.mi_infer_matmul(None, 2, shp, 2, None, 0, 0, 0, out, C.byref(n)) == INFER_ERR
    assert lb.mi_infer_matmul(shp, 9, shp, 2, None, 0, 0, 0, out, C.byref(n)) == INFER_ERR
    assert lb.mi_infer_fullconnection(shp, 2, shp, 2, None, 0, 0, 0, 0, out, None) == -2
    assert lb.mi_infer_conv2d(shp, 2, shp, 2, None, out, C.byref(n)) == -2
