"""GPU parity: every entry point of the C ABI against the CPU oracle (bit-exact for int8 outputs, bit-exact for the
fp32 outputs of the dynamic MatMul, exact scale/zero point for DynamicQuant) and against the committed golden
vectors produced by the compiled nnacl."""
import os

import numpy as np
import pytest

from mindspore_amd import kernels as K
from mindspore_amd.kernels import QuantParam as QP
from oracle import pyoracle
from oracle.pyoracle import conv_shape

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_cases.npz")


def _qps(sw, zw):
    return [QP(float(s), int(z)) for s, z in zip(np.atleast_1d(sw), np.atleast_1d(zw))]


def _mm_case(rng, m, n, k, peroc, zwnz, hb, act, bt=True, so_mul=100.0):
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w_nk = rng.integers(-128, 128, (n, k), dtype=np.int8)
    nf = n if peroc else 1
    sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
    zw = rng.integers(-10, 11, nf).astype(np.int32) if zwnz else np.zeros(nf, np.int32)
    bias = rng.integers(-5000, 5001, n).astype(np.int32) if hb else None
    sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
    so = float(sx * sw.mean() * np.sqrt(k) * so_mul)
    zo = int(rng.integers(-20, 21))
    w = w_nk if bt else np.ascontiguousarray(w_nk.T)
    return dict(a=a, w=w, bias=bias, sx=sx, zx=zx, sw=sw, zw=zw, so=so, zo=zo, act=act, b_transpose=bt)


def _gpu_matmul(case, device_tensors=False, decode_pack=True):
    kern = K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]), _qps(case["sw"], case["zw"]),
                              QP(case["so"], case["zo"]), case["b_transpose"], case["act"], decode_pack=decode_pack)
    if device_tensors:
        import torch
        out = kern.run(torch.from_numpy(case["a"]).cuda())
        torch.cuda.synchronize()
        return out.cpu().numpy(), kern
    return kern.run(case["a"]), kern


MM_SHAPES = [(1, 1, 1), (1, 64, 16), (2, 5, 7), (3, 100, 15), (4, 256, 128), (5, 260, 129), (7, 33, 1000), (8, 512, 768),
             (9, 64, 64), (31, 31, 31), (64, 64, 128), (65, 65, 130), (128, 768, 768), (129, 257, 513),
             (300, 100, 17), (500, 1030, 96), (1000, 3, 256), (2049, 1100, 64),
             # few rows against long weight rows: the deep-prefetch tile configuration (16 LDS stages)
             (17, 100, 1024), (33, 260, 2048), (64, 512, 4096), (40, 64, 1280), (20, 36, 5120),
             (65, 100, 1024), (128, 260, 2048), (100, 64, 1280),
             # more than 128 rows, few tiles and a long K: the 64 x 64 tiles on eight stages, two workgroups per CU
             (129, 260, 2048), (300, 500, 1040), (200, 4100, 1024), (384, 333, 4112),
             # too many 64 x 64 tiles for one round but not too many 64-channel x 128-row ones, K >= 2048
             (384, 4100, 2048), (1100, 1000, 2100),
             # a few hundred rows against many channels: the 256-channel x 128-row tile; two workgroups per CU on the
             # 128 x 128 tile (4224 x 2100 gives 33 x 17 of them)
             (300, 11008, 80), (512, 8196, 272), (129, 32772, 48), (4224, 2100, 144)]


@pytest.mark.parametrize("m,n,k", MM_SHAPES)
def test_matmul_shapes(orc, m, n, k):
    rng = np.random.default_rng(m * 7919 + n * 31 + k)
    orc.set_threads(16)
    for it in range(4):
        case = _mm_case(rng, m, n, k, bool(it & 1), bool(it & 2), it != 2, [0, 1, 3, 0][it], it != 3)
        got, _ = _gpu_matmul(case, device_tensors=bool(it & 1))
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (m, n, k, it, int((got != want).sum()))


@pytest.mark.parametrize("n,k", [(40, 2048), (24, 4000), (16, 5008), (9, 13008), (8200, 1040), (8196, 208),
                                 (21, 2800), (18, 6144), (13, 7008), (11, 8192), (7, 9232), (10, 10240), (6, 11008),
                                 (5, 12288), (11008, 528), (8250, 80)])
def test_decode_rows_every_stream_shape(orc, n, k):
    """1..64 activation rows (v_dot4 kernel for one row, and for two on a handle without the blocked copy; matrix-core
    kernel otherwise: one group of 16 rows up to 16, two
    groups up to 32, four up to 64, eight up to 128 against at most 4096 channels with K >= 1024) and the first row counts of
    the GEMM path, against every weight-stream shape the
    skinny path distinguishes: rows of one to six 1 KiB segments (whole rows per wave), seven to twelve (two waves
    per row, even and odd segment counts), a stream longer than the in-flight queue, few and many output channels
    (from 8192 channels on a workgroup of the matrix-core kernel owns three groups of 16 channels: 11008 channels end
    in a workgroup with one live group, 8250 in one whose live group is ragged)."""
    rng = np.random.default_rng(n * 131 + k)
    orc.set_threads(16)
    for m in list(range(1, 19)) + [23, 31, 32, 33, 40, 48, 63, 64, 65, 96, 127, 128, 129]:
        case = _mm_case(rng, m, n, k, bool(m & 1), bool(m & 2), m != 4, [0, 1, 3][m % 3])
        got, _ = _gpu_matmul(case, device_tensors=bool(m & 4))
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (m, n, k, int((got != want).sum()))
        if m == 2:  # two rows on a handle without the blocked copy: the v_dot4 kernel instead of the matrix cores
            got, _ = _gpu_matmul(case, device_tensors=True, decode_pack=False)
            assert np.array_equal(got, want), ("no blocked copy", m, n, k)


@pytest.mark.parametrize("m,n,k", [(2100, 6144, 1008), (3073, 4100, 144), (4096, 3072, 64), (2049, 6148, 400),
                                   (3072, 4096, 336)])
def test_matmul_whole_cu_tile_ragged(orc, m, n, k):
    """The 256 x 256 tile (128-byte K blocks, biased accumulators) with ragged rows, channels and K: K below one
    block, two, three and more blocks, K that ends inside a block, inside its first half, per-tensor / per-channel, zero and non-zero weight zero
    points, the generic rounding path."""
    rng = np.random.default_rng(m + n + k)
    orc.set_threads(16)
    for it in range(4):
        case = _mm_case(rng, m, n, k, bool(it & 1), bool(it & 2), it != 2, [0, 1, 3, 0][it], it != 3,
                        1e-3 if it == 3 else 100.0)
        if it == 3:
            case["bias"] = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
        got, _ = _gpu_matmul(case, device_tensors=True)
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (m, n, k, it, int((got != want).sum()))


@pytest.mark.parametrize("m,n,k", [(4352, 4096, 256), (4096, 4352, 384), (8448, 2304, 128 * 5), (2304, 8448, 256),
                                   (16640, 1024, 256), (4352, 4096, 2048)])
def test_matmul_more_full_tiles_than_cus(orc, m, n, k):
    """More full 256 x 256 tiles than CUs (272 to 297 of them: some CUs run a second tile), K a whole number of
    128-byte blocks (2, 3, 5 and 16 per tile).  Per-tensor / per-channel, zero and non-zero weight zero points, the
    generic rounding path."""
    rng = np.random.default_rng(m + 3 * n + k)
    orc.set_threads(16)
    for it in range(4):
        case = _mm_case(rng, m, n, k, bool(it & 1), bool(it & 2), it != 2, [0, 1, 3, 0][it], it != 3,
                        1e-3 if it == 3 else 100.0)
        if it == 3:
            case["bias"] = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
        got, _ = _gpu_matmul(case, device_tensors=True)
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (m, n, k, it, int((got != want).sum()))


@pytest.mark.parametrize("m,n,k", [(1408, 1408, 144), (1500, 1420, 144), (1536, 1536, 112), (1300, 1700, 400),
                                   (2050, 1030, 1168), (700, 5000, 128), (1664, 1280, 256)])
def test_matmul_128_tile_k_block_loop(orc, m, n, k):
    """The 128 x 128 tile with 128-byte K blocks (two workgroups per CU) and its neighbours: 121 tiles (below its
    range) and 144, K below one block and exactly one, two, K that ends inside a block, ragged rows and channels,
    whole tiles only; per-tensor / per-channel, zero and non-zero weight zero points, the generic rounding path."""
    rng = np.random.default_rng(m * 3 + n * 5 + k)
    orc.set_threads(16)
    for it in range(4):
        case = _mm_case(rng, m, n, k, bool(it & 1), bool(it & 2), it != 2, [0, 1, 3, 0][it], it != 3,
                        1e-3 if it == 3 else 100.0)
        if it == 3:
            case["bias"] = rng.integers(-2 ** 31, 2 ** 31 - 1, n).astype(np.int32)
        got, _ = _gpu_matmul(case, device_tensors=True)
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (m, n, k, it, int((got != want).sum()))


@pytest.mark.parametrize("rows,k,ns", [(1, 4096, (1100, 900)), (2, 1040, (64, 260, 36)), (1, 144, (8, 4, 12, 20)),
                                       (1, 11008, (300, 301)), (5, 4096, (256, 8200)), (8, 1040, (48, 16, 100)),
                                       (17, 2048, (40, 520)), (32, 400, (33, 31, 64, 5)),
                                       (40, 528, (96, 100)), (3, 64, (8, 8, 8, 8, 8))])
def test_matmul_group_equals_member_by_member(orc, rows, k, ns):
    """mi_matmul_run_group: members that share the input run as one launch (up to 32 rows, two to four members) or
    one after the other (more rows, five members); every member's output is compared with the oracle.  Members differ
    in width, quantisation granularity, weight zero points and activation."""
    import torch
    rng = np.random.default_rng(rows * 131 + k + sum(ns))
    a = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
    cases, kerns = [], []
    for i, n in enumerate(ns):
        c = _mm_case(rng, rows, n, k, bool(i & 1), i % 3 == 2, i != 1, [0, 1, 3, 0][i % 4])
        c.update(a=a, sx=sx, zx=zx)
        cases.append(c)
        kerns.append(K.MatmulInt8Kernel(c["w"], c["bias"], QP(sx, zx), _qps(c["sw"], c["zw"]), QP(c["so"], c["zo"]),
                                        c["b_transpose"], c["act"]))
    outs = K.matmul_run_group(kerns, torch.from_numpy(a).cuda())
    torch.cuda.synchronize()
    for i, c in enumerate(cases):
        want = orc.matmul_int8(**c)
        got = outs[i].cpu().numpy()
        assert np.array_equal(got, want), (rows, k, ns, i, int((got != want).sum()))


def test_matmul_generic_rounding_paths(orc):
    """Cases the fast epilogue must not take: real multiplier >= 1 (left shift), shift 0, huge bias (wrap)."""
    rng = np.random.default_rng(5)
    for m in (3, 200):
        for so_mul in (1e-4, 1e-3, 0.02):
            case = _mm_case(rng, m, 70, 40, True, True, True, 0, True, so_mul)
            case["bias"] = rng.integers(-2 ** 31, 2 ** 31 - 1, 70).astype(np.int32)
            got, kern = _gpu_matmul(case)
            assert np.array_equal(got, orc.matmul_int8(**case)), (m, so_mul)
            p = kern.params()
            mult, ls, rs = orc.requant_params(case["sx"], case["sw"], case["so"])
            assert np.array_equal(p["multiplier"], mult) and np.array_equal(p["left_shift"], ls)
            assert np.array_equal(p["right_shift"], rs)


def test_matmul_reuse_and_row_counts(orc):
    """One handle, many row counts (GEMV path, each GEMM tile choice, and back)."""
    rng = np.random.default_rng(6)
    case = _mm_case(rng, 1, 384, 256, True, False, True, 0)
    kern = K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]), _qps(case["sw"], case["zw"]),
                              QP(case["so"], case["zo"]), True, 0)
    for m in (1, 8, 9, 700, 3, 5000, 2):
        a = rng.integers(-128, 128, (m, 256), dtype=np.int8)
        case["a"] = a
        assert np.array_equal(kern.run(a), orc.matmul_int8(**case)), m


def test_handle_survives_a_failed_allocation_of_the_decode_copy(orc):
    """The blocked second copy of the weights is an optimisation: when the device has no room for it the handle is
    still created, and 2..32 rows run on the kernels that read the row-major weights."""
    from mindspore_amd import lib
    rng = np.random.default_rng(77)
    L = lib.init(0)
    n, k = 100, 300
    blocked_bytes = 256 * 512  # n and k padded to 256
    for rows in (2, 7, 32):
        c = _mm_case(rng, rows, n, k, True, True, True, 0)
        want = orc.matmul_int8(**c)
        assert L.mi_debug_fail_alloc(blocked_bytes) == 0
        try:
            got, kern = _gpu_matmul(c, device_tensors=True)
        finally:
            L.mi_debug_fail_alloc(0)
        assert np.array_equal(got, want), rows
        got2, _ = _gpu_matmul(c, device_tensors=True)  # with the copy: the matrix-core decode kernel
        assert np.array_equal(got2, want), rows
    # an allocation the handle cannot do without still fails the create, with the memory status
    assert L.mi_debug_fail_alloc(256 * 768 + 16) == 0  # the row-major packed weights
    try:
        with pytest.raises(lib.MiError) as err:
            _gpu_matmul(c)
        assert err.value.code == lib.MI_MEMORY_FAILED
    finally:
        L.mi_debug_fail_alloc(0)


def test_golden_small_cases(orc):
    g = np.load(GOLDEN)
    for i in range(int(g["mm_count"][0])):
        p = "mm%d_" % i
        sx, zx, so, zo, act, bt, hb = g[p + "meta"]
        kern = K.MatmulInt8Kernel(g[p + "w"], g[p + "bias"] if hb else None, QP(sx, int(zx)),
                                  _qps(g[p + "sw"], g[p + "zw"]), QP(so, int(zo)), bool(bt), int(act))
        assert np.array_equal(kern.run(g[p + "a"]), g[p + "c"]), p
    for i in range(int(g["cv_count"][0])):
        p = "cv%d_" % i
        sx, zx, so, zo, act, hb = g[p + "meta"]
        kh, kw, sh, sw_, dh, dw_, pu, pd, pl, pr, depthwise = [int(v) for v in g[p + "geom"]]
        w = g[p + "w"]
        kern = K.ConvolutionInt8Kernel(w, g[p + "bias"] if hb else None, QP(sx, int(zx)),
                                       _qps(g[p + "sw"], g[p + "zw"]), QP(so, int(zo)), (sh, sw_), (dh, dw_),
                                       (pu, pd, pl, pr), w.shape[0] if depthwise else 1, int(act),
                                       exact_3x3=not depthwise and (kh, kw, sh, sw_, dh, dw_) == (3, 3, 1, 1, 1, 1))
        assert np.array_equal(kern.run(g[p + "x"]), g[p + "y"]), p
    for i in range(int(g["dq_count"][0])):
        p = "dq%d_" % i
        s, z, sym = g[p + "meta"]
        q, qp = K.DynamicQuantKernel(bool(sym)).run(g[p + "x"])
        assert qp.scale == s and qp.zero_point == int(z), p
        assert np.array_equal(q, g[p + "q"]), p
    for i in range(int(g["dm_count"][0])):
        p = "dm%d_" % i
        sx, zx, act, bt, hb = g[p + "meta"]
        kern = K.MatmulDynamicInt8Kernel(g[p + "w"], g[p + "bias"] if hb else None, _qps(g[p + "sw"], g[p + "zw"]),
                                         bool(bt), int(act))
        got = kern.run(g[p + "a"], QP(sx, int(zx)))
        assert np.array_equal(got.view(np.uint32), g[p + "c"].view(np.uint32)), p


CONV_CASES = [
    (1, 5, 5, 3, 4, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    (2, 6, 7, 5, 9, (3, 3), (2, 1), (1, 1), (1, 1, 1, 1)),
    (1, 8, 8, 4, 8, (5, 3), (1, 1), (1, 1), (2, 2, 1, 1)),
    (1, 9, 9, 2, 3, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
    (1, 4, 6, 16, 5, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (2, 5, 5, 7, 6, (1, 1), (2, 2), (1, 1), (0, 0, 0, 0)),
    (1, 5, 5, 3, 10, (1, 1), (1, 1), (1, 1), (1, 1, 1, 1)),
    (1, 6, 6, 3, 4, (1, 1), (2, 2), (1, 1), (1, 0, 1, 0)),
    (1, 7, 5, 3, 17, (2, 2), (1, 1), (1, 1), (0, 0, 0, 0)),
    (1, 40, 40, 32, 64, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1)),
    (3, 28, 28, 64, 300, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (1, 30, 30, 24, 16, (7, 7), (2, 2), (1, 1), (3, 3, 3, 3)),
    # short contraction (K <= 64): gathered straight from the image
    (2, 13, 11, 4, 96, (4, 4), (1, 1), (1, 1), (1, 2, 2, 1)),
    (1, 9, 9, 3, 128, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1)),
    (1, 9, 9, 1, 36, (5, 5), (1, 1), (2, 2), (4, 4, 4, 4)),
    (1, 64, 48, 3, 32, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    # 16-channel-aligned images with more than 128 output pixels: the GEMM gathers from the image, no im2col buffer
    (1, 33, 31, 32, 20, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
    (2, 30, 30, 80, 36, (1, 1), (2, 2), (1, 1), (1, 1, 1, 1)),
    (1, 20, 20, 16, 8, (5, 5), (1, 1), (1, 1), (2, 2, 2, 2)),
    (1, 20, 24, 16, 8, (3, 1), (1, 2), (1, 1), (1, 1, 0, 0)),
    (2, 96, 96, 16, 132, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    (1, 23, 17, 48, 64, (2, 4), (1, 1), (3, 2), (3, 3, 4, 4)),
]


def _conv_case(rng, b, ih, iw, ic, oc, kernel, stride, dil, pad, peroc, zwnz, hb, act, dw=False):
    shape = conv_shape(b, ih, iw, ic, oc, kernel, stride, dil, pad)
    x = rng.integers(-128, 128, (b, ih, iw, ic), dtype=np.int8)
    w = rng.integers(-128, 128, (oc, kernel[0], kernel[1]) if dw else (oc, kernel[0], kernel[1], ic), dtype=np.int8)
    nf = oc if peroc else 1
    sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
    zw = rng.integers(-10, 11, nf).astype(np.int32) if zwnz else np.zeros(nf, np.int32)
    bias = rng.integers(-3000, 3001, oc).astype(np.int32) if hb else None
    sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
    kdim = kernel[0] * kernel[1] * (1 if dw else ic)
    so = float(sx * sw.mean() * np.sqrt(kdim) * 100)
    zo = int(rng.integers(-20, 21))
    return dict(x=x, w=w, bias=bias, shape=shape, sx=sx, zx=zx, sw=sw, zw=zw, so=so, zo=zo, act=act)


def _gpu_conv(case, stride, dil, pad, group=1, device_tensors=False, exact_3x3=False):
    kern = K.ConvolutionInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]), _qps(case["sw"], case["zw"]),
                                   QP(case["so"], case["zo"]), stride, dil, pad, group, case["act"],
                                   exact_3x3=exact_3x3)
    if device_tensors:
        import torch
        out = kern.run(torch.from_numpy(case["x"]).cuda())
        torch.cuda.synchronize()
        return out.cpu().numpy()
    return kern.run(case["x"])


@pytest.mark.parametrize("idx", range(len(CONV_CASES)))
def test_conv_cases(orc, idx):
    rng = np.random.default_rng(900 + idx)
    orc.set_threads(16)
    b, ih, iw, ic, oc, kernel, stride, dil, pad = CONV_CASES[idx]
    for it in range(4):
        case = _conv_case(rng, b, ih, iw, ic, oc, kernel, stride, dil, pad, bool(it & 1), bool(it & 2), it != 3,
                          [0, 1, 3, 0][it])
        got = _gpu_conv(case, stride, dil, pad, 1, device_tensors=bool(it & 1))
        want = orc.conv_int8(**case)
        assert np.array_equal(got, want), (idx, it, int((got != want).sum()))
        if it == 2 and pyoracle.Reference.available():  # and the compiled nnacl itself
            r = pyoracle.reference()
            r.threads = 16
            assert np.array_equal(got, r.conv_int8(**case)), (idx, "compiled nnacl")


DW_CASES = [
    (1, 6, 6, 5, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (2, 7, 5, 8, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    (1, 9, 9, 3, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
    (1, 56, 56, 96, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (1, 15, 18, 16, (5, 5), (1, 2), (1, 1), (2, 2, 2, 2)),
    (2, 11, 9, 32, (3, 3), (2, 1), (2, 2), (2, 2, 2, 2)),
    (1, 4, 4, 48, (3, 3), (1, 1), (1, 1), (2, 2, 2, 2)),
    (1, 28, 28, 24, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),   # 8 channels per thread
    (2, 10, 12, 40, (5, 5), (2, 2), (1, 1), (2, 2, 2, 2)),
]


@pytest.mark.parametrize("idx", range(len(DW_CASES)))
def test_depthwise_cases(orc, idx):
    rng = np.random.default_rng(950 + idx)
    orc.set_threads(16)
    b, ih, iw, ch, kernel, stride, dil, pad = DW_CASES[idx]
    for it in range(4):
        case = _conv_case(rng, b, ih, iw, ch, ch, kernel, stride, dil, pad, bool(it & 1), bool(it & 2), it != 3,
                          [0, 1, 3, 0][it], dw=True)
        got = _gpu_conv(case, stride, dil, pad, ch, device_tensors=bool(it & 1))
        assert np.array_equal(got, orc.conv_dw_int8(**case)), (idx, it)


def test_conv_declines_what_the_provider_must_not_claim():
    w = np.zeros((8, 3, 3, 4), np.int8)
    with pytest.raises(K._lib.MiError) as e:
        K.ConvolutionInt8Kernel(w, None, QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0), (1, 1), (1, 1), (1, 1, 1, 1))
    assert e.value.code == K._lib.MI_NOT_SUPPORT
    with pytest.raises(K._lib.MiError) as e:  # grouped, not depthwise
        K.ConvolutionInt8Kernel(np.zeros((8, 3, 3), np.int8), None, QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0), (2, 2),
                                group=4)
    assert e.value.code == K._lib.MI_NOT_SUPPORT


@pytest.mark.parametrize("shape", [(1, 14, 14, 64, 96), (2, 9, 11, 5, 12), (1, 56, 56, 64, 64), (1, 7, 7, 3, 8),
                                   (4, 64, 64, 16, 128), (4, 64, 66, 16, 40), (32, 56, 56, 16, 8)])
def test_dense_3x3_stride_1_as_the_exact_convolution(orc, shape):
    """With MI_CONV_3X3_EXACT the library takes the convolutions it otherwise leaves to the reference's Winograd
    kernel and computes ConvInt8 on them, the kernel the reference itself selects on ARM64 with dot product
    (convolution_int8_creator.cc:81-94): compared with nnacl's ConvInt8 on the same inputs."""
    b, ih, iw, ic, oc = shape
    rng = np.random.default_rng(ih * 100 + ic)
    orc.set_threads(16)
    for it in range(4):
        pad = [(1, 1, 1, 1), (0, 0, 0, 0), (1, 0, 0, 1), (2, 2, 2, 2)][it]
        case = _conv_case(rng, b, ih, iw, ic, oc, (3, 3), (1, 1), (1, 1), pad, bool(it & 1), bool(it & 2), it != 3,
                          [0, 1, 3, 0][it])
        got = _gpu_conv(case, (1, 1), (1, 1), pad, 1, device_tensors=bool(it & 1), exact_3x3=True)
        want = orc.conv_int8_as_arm64_sdot(**case)
        assert got.shape == want.shape and np.array_equal(got, want), (shape, it)
        if it == 0 and pyoracle.Reference.available():  # the compiled ConvInt8 itself
            r = pyoracle.reference()
            r.threads = 16
            assert np.array_equal(got, r.conv_int8_as_arm64_sdot(**case)), (shape, "compiled nnacl")
    with pytest.raises(K._lib.MiError) as e:
        _gpu_conv(case, (1, 1), (1, 1), pad, 1)
    assert e.value.code == K._lib.MI_NOT_SUPPORT


def _dq_inputs():
    rng = np.random.default_rng(300)
    xs = [rng.standard_normal(5000).astype(np.float32), rng.standard_normal((37, 91)).astype(np.float32) * 5 + 3,
          np.zeros(700, np.float32), np.full(1000, 2.5, np.float32), np.array([1.0], np.float32),
          rng.uniform(-1e-3, 1e-3, 4096).astype(np.float32), np.linspace(-7.5, 9.25, 3001, dtype=np.float32),
          (rng.standard_normal(2048) * 1e6).astype(np.float32), rng.standard_normal(1 << 20).astype(np.float32),
          rng.standard_normal(4099 * 257).astype(np.float32) * 3]
    sp = rng.standard_normal(3000).astype(np.float32)
    sp[5], sp[77], sp[900] = np.nan, 12.5, -13.25
    xs.append(sp)
    xs.append(np.array([np.inf, -np.inf, 1.0, -2.0, 3e38, -3e38, np.nan, 0.0] * 9, np.float32))
    # both sides of the size up to which one workgroup does the whole tensor in one launch, and a few decode rows
    xs += [rng.standard_normal(24576).astype(np.float32), rng.standard_normal(24577).astype(np.float32) * 2 - 1,
           rng.standard_normal((2, 11008)).astype(np.float32), rng.standard_normal(24575).astype(np.float32),
           rng.standard_normal(3).astype(np.float32), rng.standard_normal((8, 4096)).astype(np.float32)]
    return xs


def test_dynamic_quant(orc):
    import torch
    for i, x in enumerate(_dq_inputs()):
        for sym in (False, True):
            kern = K.DynamicQuantKernel(sym)
            q_ref, s_ref, z_ref = orc.dynamic_quant(x, sym)
            q, qp = kern.run(x)
            assert qp.scale == s_ref and qp.zero_point == z_ref, (i, sym, qp, s_ref, z_ref)
            assert np.array_equal(q, q_ref), (i, sym)
            xt = torch.from_numpy(x).cuda()
            q2, qp2 = kern.run(xt)
            assert qp2 == qp and np.array_equal(q2.cpu().numpy(), q_ref)
            # unaligned device pointer
            if x.size > 8:
                q3, qp3 = kern.run(xt.reshape(-1)[1:])
                q3r, s3, z3 = orc.dynamic_quant(x.reshape(-1)[1:], sym)
                assert qp3.scale == s3 and qp3.zero_point == z3 and np.array_equal(q3.cpu().numpy(), q3r)


def test_dynamic_matmul(orc):
    import torch
    rng = np.random.default_rng(401)
    orc.set_threads(16)
    for it, (m, n, k) in enumerate([(1, 1, 1), (5, 9, 17), (33, 70, 64), (130, 65, 300), (9, 256, 1000),
                                    (700, 300, 129), (64, 2304, 768), (4100, 4096, 400), (4097, 4100, 208),
                                    # fp32 output on the 128-tile K-block loop: at most one tile per CU, K >= 2048,
                                    # 768 tiles and more; and 306 tiles, which stay on the 64-byte-step loop
                                    (1500, 1420, 144), (1300, 1290, 2064), (4100, 3000, 144), (2100, 2304, 208),
                                    # few tiles and a long K: 64 x 64 tiles on eight stages
                                    (260, 516, 1100), (129, 100, 2048), (520, 2100, 2064)]):
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        w = rng.integers(-128, 128, (n, k), dtype=np.int8)
        nf = n if it & 1 else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = np.full(nf, 0 if it & 2 else int(rng.integers(-5, 6)), np.int32)
        bias = rng.standard_normal(n).astype(np.float32) if it & 4 else None
        sx, zx, act = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128)), [0, 1, 3][it % 3]
        bt = it != 3
        wmem = w if bt else np.ascontiguousarray(w.T)
        kern = K.MatmulDynamicInt8Kernel(wmem, bias, _qps(sw, zw), bt, act)
        want = orc.dynamic_matmul(a, wmem, bias, sx, zx, sw, zw, act, bt)
        got = kern.run(a, QP(sx, zx))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (it, m, n, k)
        got2 = kern.run(torch.from_numpy(a).cuda(), QP(sx, zx)).cpu().numpy()
        assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n,k", [(4096, 4096), (8200, 1040), (11008, 528), (300, 11008), (21, 2800), (7, 100),
                                 (8250, 80), (515, 3000)])
def test_dynamic_matmul_decode_rows(orc, n, k):
    """1..64 rows of the dynamic-quant MatMul take the decode kernels with the fp32 epilogue (one and three
    channel groups per workgroup, ragged channels and K, one, two, four and eight groups of activation rows); 129
    rows, 65..128 against many channels or a short K, and a handle without the blocked weight copy take the GEMM tiles.  Per-tensor and per-channel weight scales, a weight zero
    point, bias, every activation; input parameters by value, from device memory, and one scale per row."""
    import torch
    rng = np.random.default_rng(n * 7 + k)
    orc.set_threads(16)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    for it, m in enumerate([1, 2, 3, 5, 8, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 129]):
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        nf = n if it & 1 else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = np.full(nf, 0 if it & 2 else int(rng.integers(-5, 6)), np.int32)
        bias = rng.standard_normal(n).astype(np.float32) if it % 3 else None
        sx, zx, act = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128)), [0, 1, 3][it % 3]
        kern = K.MatmulDynamicInt8Kernel(w, bias, _qps(sw, zw), True, act)
        want = orc.dynamic_matmul(a, w, bias, sx, zx, sw, zw, act, True)
        got = kern.run(torch.from_numpy(a).cuda(), QP(sx, zx)).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (m, n, k, "by value")
        if it % 4 == 0:  # the same through a handle without the blocked copy
            plain = K.MatmulDynamicInt8Kernel(w, bias, _qps(sw, zw), True, act, decode_pack=False)
            got = plain.run(torch.from_numpy(a).cuda(), QP(sx, zx)).cpu().numpy()
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (m, n, k, "no blocked copy")
        if it % 2 == 0:  # one input scale per row (the zero point is that of the first row, as in the reference)
            sxr = rng.uniform(0.01, 0.1, m).astype(np.float32)
            want_r = orc.dynamic_matmul_rows(a, w, bias, sxr, zx, sw, zw, act)
            got_r = kern.run(a, [QP(float(s), zx) for s in sxr])
            assert np.array_equal(got_r.view(np.uint32), want_r.view(np.uint32)), (m, n, k, "per row")


@pytest.mark.parametrize("rows,k,ns", [(1, 4096, (1100, 900)), (2, 1040, (64, 260, 36)), (1, 144, (8, 4, 12, 20)),
                                       (5, 4096, (256, 8200)), (8, 1040, (48, 16, 100)), (17, 2048, (40, 520)),
                                       (32, 400, (33, 31, 64, 5)), (40, 528, (96, 100)), (3, 64, (8, 8, 8, 8, 8))])
def test_dynamic_matmul_group_equals_member_by_member(orc, rows, k, ns):
    """mi_dynmm_run_group: dynamic MatMuls that share their input run as one launch (up to 32 rows, two to four
    members) or one after the other (more rows, five members); every member's fp32 output is compared with the oracle,
    for an input scale given by value, read from the block DynamicQuant left on the device, and one scale per row."""
    import torch
    rng = np.random.default_rng(rows * 137 + k + sum(ns))
    orc.set_threads(16)
    x = (rng.standard_normal((rows, k)) * 2).astype(np.float32)
    cases, kerns = [], []
    for i, n in enumerate(ns):
        w = rng.integers(-128, 128, (n, k), dtype=np.int8)
        nf = n if i & 1 else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = np.full(nf, 0 if i % 3 else int(rng.integers(-5, 6)), np.int32)
        bias = rng.standard_normal(n).astype(np.float32) if i != 1 else None
        act = [0, 1, 3, 0][i % 4]
        cases.append((w, bias, sw, zw, act))
        kerns.append(K.MatmulDynamicInt8Kernel(w, bias, _qps(sw, zw), True, act))
    # by value
    a = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    sx, zx = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128))
    outs = K.dynmm_run_group(kerns, torch.from_numpy(a).cuda(), in_quant=QP(sx, zx))
    torch.cuda.synchronize()
    for i, (w, bias, sw, zw, act) in enumerate(cases):
        want = orc.dynamic_matmul(a, w, bias, sx, zx, sw, zw, act, True)
        assert np.array_equal(outs[i].cpu().numpy().view(np.uint32), want.view(np.uint32)), (rows, k, ns, i, "by value")
    # chained behind DynamicQuant, per tensor and per row
    dq = K.DynamicQuantKernel(False)
    q, _ = dq.run(torch.from_numpy(x).cuda(), fetch_params=False)
    outs = K.dynmm_run_group(kerns, q, params_dev=dq.device_params())
    torch.cuda.synchronize()
    q_ref, s_ref, z_ref = orc.dynamic_quant(x)
    for i, (w, bias, sw, zw, act) in enumerate(cases):
        want = orc.dynamic_matmul(q_ref, w, bias, s_ref, z_ref, sw, zw, act, True)
        assert np.array_equal(outs[i].cpu().numpy().view(np.uint32), want.view(np.uint32)), (rows, k, ns, i, "chained")
    dqr = K.DynamicQuantKernel(True)
    qr, row_params = dqr.run_rows(torch.from_numpy(x).cuda())
    outs = K.dynmm_run_group(kerns, qr, row_params=row_params)
    torch.cuda.synchronize()
    qr_ref, sr_ref, zr_ref = orc.dynamic_quant_segments(x, True)
    for i, (w, bias, sw, zw, act) in enumerate(cases):
        want = orc.dynamic_matmul_rows(qr_ref, w, bias, sr_ref.astype(np.float32), int(zr_ref[0]), sw, zw, act)
        assert np.array_equal(outs[i].cpu().numpy().view(np.uint32), want.view(np.uint32)), (rows, k, ns, i, "per row")


def test_dynamic_quant_chained_into_matmul(orc):
    """DynamicQuant -> dynamic MatMul with the scale / zero point handed over in device memory."""
    import torch
    rng = np.random.default_rng(402)
    x = (rng.standard_normal((200, 96)) * 2).astype(np.float32)
    w = rng.integers(-127, 128, (80, 96), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, 80).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(80).astype(np.float32)
    dq = K.DynamicQuantKernel(False)
    mm = K.MatmulDynamicInt8Kernel(w, bias, _qps(sw, np.zeros(80, np.int32)))
    q, _ = dq.run(torch.from_numpy(x).cuda(), fetch_params=False)
    y = mm.run(q, params_dev=dq.device_params())
    torch.cuda.synchronize()
    q_ref, s, z = orc.dynamic_quant(x)
    want = orc.dynamic_matmul(q_ref, w, bias, s, z, sw, np.zeros(80, np.int32))
    assert np.array_equal(q.cpu().numpy(), q_ref)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("rows,k,n", [(1, 16, 24), (5, 7, 24), (37, 100, 24), (64, 768, 24), (130, 1030, 24),
                                      (3, 5000, 24),
                                      # enough 128 x 128 tiles for the K-block loop: full and ragged tiles of the
                                      # general fp32 epilogue with one input scale per row
                                      (1500, 272, 1420)])
def test_dynamic_quant_per_row_and_matmul(orc, rows, k, n):
    """Per-channel activation quantisation (one scale per row) feeding the dynamic MatMul with per-row input scales,
    host path and device-chained path, symmetric (what the converter emits) and asymmetric."""
    import torch
    rng = np.random.default_rng(rows * 1000 + k)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[rng.random((rows, k)) < 0.01] *= 8
    if rows > 2:
        x[1] = 0.25          # constant row: range 0 -> the 0.01 fallback
        x[2, 0] = np.inf     # +inf dominates the row's max
    orc.set_threads(16)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    mm = K.MatmulDynamicInt8Kernel(w, bias, _qps(sw, np.zeros(n, np.int32)))
    for symmetric in (True, False):
        want_q, want_s, want_z = orc.dynamic_quant_segments(x, symmetric)
        dq = K.DynamicQuantKernel(symmetric)
        got_q, qps = dq.run_rows(x)
        assert np.array_equal(got_q, want_q)
        assert [p.scale for p in qps] == list(want_s) and [p.zero_point for p in qps] == list(want_z)
        want_c = orc.dynamic_matmul_rows(want_q, w, bias, want_s.astype(np.float32), int(want_z[0]), sw,
                                         np.zeros(n, np.int32))
        got_c = mm.run(got_q, qps)
        assert np.array_equal(got_c.view(np.uint32), want_c.view(np.uint32))
        xq, params = dq.run_rows(torch.from_numpy(x).cuda())
        got_dev = mm.run(xq, row_params=params)
        torch.cuda.synchronize()
        assert np.array_equal(xq.cpu().numpy(), want_q)
        assert np.array_equal(got_dev.cpu().numpy().view(np.uint32), want_c.view(np.uint32))


def test_error_paths():
    """Invalid descriptors and arguments come back as Lite's status codes with a message, before anything is launched."""
    import ctypes as C
    import torch
    lib = K._lib
    L = lib.init()
    assert L.mi_matmul_run(None, None, 1, None, None) == lib.MI_NULL_PTR
    with pytest.raises(lib.MiError) as e:
        K.MatmulInt8Kernel(np.zeros((4, 8), np.int8), None, QP(0.1, 0), [QP(0.1, 0)] * 3, QP(0.1, 0))
    assert e.value.code == lib.MI_PARAM_INVALID
    with pytest.raises(TypeError):
        K.MatmulInt8Kernel(np.zeros((4, 8), np.int8), np.zeros(4, np.float32), QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0))
    # descriptors
    scales, zps = (C.c_double * 4)(0.1, 0.1, 0.1, 0.1), (C.c_int32 * 4)(0, 0, 0, 0)
    w = np.zeros((4, 8), np.int8)
    h = C.c_void_p()
    for bad in (lib.MatmulDesc(0, 4, 1, 0, 0.1, 0, 0.1, 0, 1, scales, zps),      # deep 0
                lib.MatmulDesc(8, -1, 1, 0, 0.1, 0, 0.1, 0, 1, scales, zps),     # negative col
                lib.MatmulDesc(8, 4, 1, 2, 0.1, 0, 0.1, 0, 1, scales, zps),      # activation 2 (sigmoid) unsupported
                lib.MatmulDesc(8, 4, 1, 0, 0.1, 0, 0.1, 0, 3, scales, zps)):     # 3 filter params for 4 channels
        assert L.mi_matmul_create(C.byref(bad), w.ctypes.data, None, C.byref(h)) == lib.MI_PARAM_INVALID
        assert h.value is None and L.mi_last_error() != b""
    assert L.mi_matmul_create(C.byref(lib.MatmulDesc(8, 4, 1, 0, 0.1, 0, 0.1, 0, 1, None, None)), w.ctypes.data, None,
                              C.byref(h)) == lib.MI_NULL_PTR
    assert L.mi_dynmm_create(C.byref(lib.DynmmDesc(8, 4, 1, 7, 1, scales, zps)), w.ctypes.data, None,
                             C.byref(h)) == lib.MI_PARAM_INVALID
    # runs
    kern = K.MatmulInt8Kernel(w, None, QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0))
    a = torch.zeros((2, 8), dtype=torch.int8, device="cuda")
    c = torch.zeros((2, 4), dtype=torch.int8, device="cuda")
    assert L.mi_matmul_run(kern._h, a.data_ptr(), -1, c.data_ptr(), None) == lib.MI_PARAM_INVALID
    assert L.mi_matmul_run(kern._h, a.data_ptr(), 0, c.data_ptr(), None) == lib.MI_OK          # empty batch: nothing to do
    assert L.mi_matmul_run(kern._h, None, 2, c.data_ptr(), None) == lib.MI_NULL_PTR
    dq = K.DynamicQuantKernel(False)
    assert L.mi_dynquant_run(dq._h, None, 0, None, None) == lib.MI_OK                            # empty tensor
    assert L.mi_dynquant_run(dq._h, None, 16, None, None) == lib.MI_NULL_PTR
    assert L.mi_dynquant_run(dq._h, a.data_ptr(), -4, c.data_ptr(), None) == lib.MI_PARAM_INVALID
    assert L.mi_dynquant_run_segments(dq._h, a.data_ptr(), 0, 8, c.data_ptr(), c.data_ptr(), None) == lib.MI_PARAM_INVALID
    # convolution: declined shapes are MI_NOT_SUPPORT (the provider falls back), broken ones MI_PARAM_INVALID
    with pytest.raises(lib.MiError) as e:
        K.ConvolutionInt8Kernel(np.zeros((8, 3, 3, 4), np.int8), None, QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0),
                                (0, 1), (1, 1), (0, 0, 0, 0), 1, 0)
    assert e.value.code == lib.MI_PARAM_INVALID
    conv = K.ConvolutionInt8Kernel(np.zeros((8, 1, 1, 4), np.int8), None, QP(0.1, 0), [QP(0.1, 0)], QP(0.1, 0),
                                   (1, 1), (1, 1), (0, 0, 0, 0), 1, 0)
    x = torch.zeros((1, 5, 5, 4), dtype=torch.int8, device="cuda")
    y = torch.zeros((1, 5, 5, 8), dtype=torch.int8, device="cuda")
    assert L.mi_conv_run(conv._h, x.data_ptr(), 1, 0, 5, y.data_ptr(), None) == lib.MI_PARAM_INVALID
    assert L.mi_conv_run(conv._h, x.data_ptr(), 1, 5, 5, None, None) == lib.MI_NULL_PTR

def test_first_decode_call_inside_a_graph_capture(orc):
    """All weight packing happens at create time, so the very first call of a handle may come under stream capture
    and runs the decode kernel it would run eagerly: the capture stays valid and every replay is right.  A handle
    created without the decode pack takes the same row counts on the GEMM tiles, with the same results."""
    import torch
    rng = np.random.default_rng(77)
    for k, decode_pack in ((512, True), (512, False), (500, True)):   # 500: the run also pads the activation rows
        case = _mm_case(rng, 8, 200, k, True, False, True, 0)
        kern = K.MatmulInt8Kernel(case["w"], case["bias"], QP(case["sx"], case["zx"]), _qps(case["sw"], case["zw"]),
                                  QP(case["so"], case["zo"]), True, 0, decode_pack=decode_pack)
        kern.reserve(8)   # ReSize(): the padded-row workspace exists before the capture
        a = torch.from_numpy(case["a"]).cuda()
        out = torch.zeros((8, 200), dtype=torch.int8, device="cuda")
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=st):
                kern.run(a, out=out)
        torch.cuda.synchronize()
        for rep in range(3):
            a.copy_(torch.from_numpy(rng.integers(-128, 128, (8, k), dtype=np.int8)))
            out.zero_()
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            case["a"] = a.cpu().numpy()
            want = orc.matmul_int8(**case)
            assert np.array_equal(out.cpu().numpy(), want), (k, decode_pack, rep)
            assert np.array_equal(kern.run(a).cpu().numpy(), want)
        for m in (3, 17, 32, 2, 40):   # every decode row class on this handle, eager
            case["a"] = rng.integers(-128, 128, (m, k), dtype=np.int8)
            assert np.array_equal(kern.run(case["a"]), orc.matmul_int8(**case)), (k, decode_pack, m)


def test_device_memory_entry_points(orc):
    """mi_device_malloc / mi_copy_to_device / mi_copy_to_host / mi_device_free: what a provider keeps a tensor in HBM
    with.  A buffer from them feeds a kernel launch like any device pointer."""
    import ctypes as C
    lib = K._lib
    L = lib.init()
    p = C.c_void_p()
    assert L.mi_device_malloc(0, C.byref(p)) == lib.MI_PARAM_INVALID and p.value is None
    assert L.mi_device_malloc(64, None) == lib.MI_NULL_PTR
    assert L.mi_device_free(None) == lib.MI_OK
    assert L.mi_copy_to_device(None, None, 0, None) == lib.MI_OK
    assert L.mi_copy_to_device(None, None, 8, None) == lib.MI_NULL_PTR
    assert L.mi_copy_to_host(None, None, 8, None) == lib.MI_NULL_PTR
    rng = np.random.default_rng(21)
    m, k, n = 7, 200, 52
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    bias = rng.integers(-3000, 3000, n).astype(np.int32)
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    kern = K.MatmulInt8Kernel(w, bias, QP(0.03, 4), [QP(s, 0) for s in sw], QP(0.07, -2))
    a_dev, c_dev = C.c_void_p(), C.c_void_p()
    assert L.mi_device_malloc(a.nbytes, C.byref(a_dev)) == lib.MI_OK and a_dev.value
    assert L.mi_device_malloc(m * n, C.byref(c_dev)) == lib.MI_OK and c_dev.value
    assert L.mi_copy_to_device(a_dev, a.ctypes.data, a.nbytes, None) == lib.MI_OK
    back = np.empty_like(a)
    assert L.mi_copy_to_host(back.ctypes.data, a_dev, a.nbytes, None) == lib.MI_OK and np.array_equal(back, a)
    assert L.mi_matmul_run(kern._h, a_dev, m, c_dev, None) == lib.MI_OK
    assert L.mi_stream_synchronize(None) == lib.MI_OK
    got = np.empty((m, n), np.int8)
    assert L.mi_copy_to_host(got.ctypes.data, c_dev, got.nbytes, None) == lib.MI_OK
    want = orc.matmul_int8(a, w, bias, 0.03, 4, sw, np.zeros(n, np.int32), 0.07, -2, 0, True)
    assert np.array_equal(got, want)
    assert L.mi_device_free(a_dev) == lib.MI_OK and L.mi_device_free(c_dev) == lib.MI_OK
