"""Pins the oracle's MatMul / Conv / depthwise / DynamicQuant / dynamic-MatMul restatements against
(1) exact int64 / float32 closed forms on small shapes (tests/closed_forms.py),
(2) the compiled nnacl driven through the Lite wrappers' call sequences (oracle/_ref), on many random shapes,
(3) known answers taken from the reference's own unit tests."""
import numpy as np
import pytest

from oracle.pyoracle import ACT_NONE, ACT_RELU, ACT_RELU6, conv_shape
from tests import closed_forms as cf


def _mm_case(rng, m, n, k, peroc, zw_nonzero, has_bias, act, b_transpose=True):
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w_nk = rng.integers(-128, 128, (n, k), dtype=np.int8)
    nf = n if peroc else 1
    sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
    zw = rng.integers(-10, 11, nf).astype(np.int32) if zw_nonzero else np.zeros(nf, np.int32)
    bias = rng.integers(-5000, 5001, n).astype(np.int32) if has_bias else None
    sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
    so = float(sx * sw.mean() * np.sqrt(k) * 40)
    zo = int(rng.integers(-20, 21))
    w = w_nk if b_transpose else np.ascontiguousarray(w_nk.T)
    return dict(a=a, w=w, bias=bias, sx=sx, zx=zx, sw=sw, zw=zw, so=so, zo=zo, act=act, b_transpose=b_transpose), w_nk


MM_SHAPES = [(1, 1, 1), (3, 5, 7), (4, 4, 16), (5, 9, 17), (8, 12, 33), (13, 10, 64), (2, 31, 100)]


@pytest.mark.parametrize("m,n,k", MM_SHAPES)
@pytest.mark.parametrize("peroc", [False, True])
@pytest.mark.parametrize("zw_nonzero", [False, True])
def test_matmul_closed_form(orc, m, n, k, peroc, zw_nonzero):
    rng = np.random.default_rng(m * 1000 + n * 10 + k + peroc * 7 + zw_nonzero * 3)
    for act in (ACT_NONE, ACT_RELU, ACT_RELU6):
        for has_bias in (True, False):
            for bt in (True, False):
                case, w_nk = _mm_case(rng, m, n, k, peroc, zw_nonzero, has_bias, act, bt)
                got = orc.matmul_int8(**case)
                want = cf.matmul_int8(case["a"], w_nk, case["bias"], case["sx"], case["zx"], case["sw"], case["zw"],
                                      case["so"], case["zo"], act)
                assert np.array_equal(got, want)


def test_matmul_multiplier_above_one_and_wrap(orc, ref):
    # real multiplier >= 1 -> left shift > 0; a huge bias makes acc * 2^ls wrap in int32
    rng = np.random.default_rng(11)
    a = rng.integers(-128, 128, (6, 40), dtype=np.int8)
    w = rng.integers(-128, 128, (9, 40), dtype=np.int8)
    bias = np.array([2 ** 30, -2 ** 30, 2 ** 31 - 1, -2 ** 31, 0, 5, 7, 2 ** 29, -2 ** 29], np.int32)
    for so in (1e-6, 1e-5, 3e-4):
        got = orc.matmul_int8(a, w, bias, 0.05, 3, [0.02], [2], so, -7)
        want = cf.matmul_int8(a, w, bias, 0.05, 3, [0.02], [2], so, -7, 0)
        assert np.array_equal(got, want)
        assert np.array_equal(got, ref.matmul_int8(a, w, bias, 0.05, 3, [0.02], [2], so, -7))


def test_matmul_vs_nnacl_random(orc, ref):
    rng = np.random.default_rng(12)
    for it in range(60):
        m, n, k = (int(rng.integers(1, 40)), int(rng.integers(1, 40)), int(rng.integers(1, 130)))
        case, _ = _mm_case(rng, m, n, k, bool(it & 1), bool(it & 2), bool(it & 4), [0, 1, 3][it % 3], bool(it & 8))
        ref.threads = 1 + it % 4
        assert np.array_equal(orc.matmul_int8(**case), ref.matmul_int8(**case)), (m, n, k, it)


def _quant_process(lo, hi):
    """QuantProcess of the reference's test (matmul_int8_tests.cc:40-46): float scale, truncated zero point."""
    scale = np.float32(np.float32(hi - lo) / np.float32(255))
    zp = int(np.float32(127) - np.float32(hi) / scale)
    return scale, zp


def _quantize(x, scale, zp):
    q = cf.round_half_away((x.astype(np.float32) / scale + np.float32(zp)).astype(np.float64))
    return np.clip(q, -128, 127).astype(np.int8)


def test_matmul_reference_unit_test_vectors(orc):
    """TestMatmulInt8.mmtest1 of the reference (mindspore/lite/test/ut/src/runtime/kernel/arm/int8/
    matmul_int8_tests.cc:83-145): same float data, same quantisation of inputs, same acceptance criterion
    (dequantised output within mean-abs 0.3 of `correct`)."""
    a = np.array([6.583835634764597, 11.337275140963907, -4.125256949459629, 10.994337291530833, 19.086065139532636,
                  3.620842999158455, 13.167624585590346, -18.326739299407755, 14.877693740734841,
                  -17.092677920571653, 19.24147072807235, -15.14805323833401, -18.075654829688737,
                  -0.9164404591894204, -3.836646280336332, -10.870298671273918], np.float32).reshape(2, 8)
    b = np.array([0.3651070698591563, -0.5856943921727129, -0.7472032663840145, 0.9489992871641959,
                  -0.8179490270358738, -0.873058811259344, 0.39876672713807215, -0.1816769383004213,
                  -0.13584645926733696, -0.7614673836659709, -0.2535825872616164, -0.05265760030895916,
                  0.28558728305658754, 0.15404213943520118, -0.1634824450738006, -0.5068199082730189,
                  -0.026961256849111326, -0.1508441942453307, 0.9375335677537737, 0.3304690744194263,
                  -0.5091563780251127, 0.029887336278646925, -0.39540496207319276, 0.46094065001445084],
                 np.float32).reshape(3, 8)
    correct = np.array([-0.912632942, 4.08398056, -25.385608673, 2.720281124, 7.745952606, 20.893184662],
                       np.float32).reshape(2, 3)
    sa, za = _quant_process(-20, 20)
    sb, zb = _quant_process(-1, 1)
    sc, zc = _quant_process(-30, 30)
    out = orc.matmul_int8(_quantize(a, sa, za), _quantize(b, sb, zb), None, float(sa), za, [float(sb)], [zb],
                          float(sc), zc)
    deq = sc * (out.astype(np.float32) - zc)
    assert np.abs(deq - correct).mean() <= 0.3


CONV_CASES = [
    # b, ih, iw, ic, oc, k, stride, dil, pad(u,d,l,r)
    (1, 5, 5, 3, 4, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    (2, 6, 7, 5, 9, (3, 3), (2, 1), (1, 1), (1, 1, 1, 1)),
    (1, 8, 8, 4, 8, (5, 3), (1, 1), (1, 1), (2, 2, 1, 1)),
    (1, 9, 9, 2, 3, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
    (1, 4, 6, 16, 5, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (2, 5, 5, 7, 6, (1, 1), (2, 2), (1, 1), (0, 0, 0, 0)),
    (1, 5, 5, 3, 10, (1, 1), (1, 1), (1, 1), (1, 1, 1, 1)),  # padded 1x1: zero-filled gather quirk
    (1, 6, 6, 3, 4, (1, 1), (2, 2), (1, 1), (1, 0, 1, 0)),
    (1, 7, 5, 3, 17, (2, 2), (1, 1), (1, 1), (0, 0, 0, 0)),
    (1, 3, 3, 1, 1, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
]


def _conv_case(rng, b, ih, iw, ic, oc, kernel, stride, dil, pad, peroc, zw_nonzero, has_bias, act, dw=False):
    shape = conv_shape(b, ih, iw, ic, oc, kernel, stride, dil, pad)
    x = rng.integers(-128, 128, (b, ih, iw, ic), dtype=np.int8)
    wshape = (oc, kernel[0], kernel[1]) if dw else (oc, kernel[0], kernel[1], ic)
    w = rng.integers(-128, 128, wshape, dtype=np.int8)
    nf = oc if peroc else 1
    sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
    zw = rng.integers(-10, 11, nf).astype(np.int32) if zw_nonzero else np.zeros(nf, np.int32)
    bias = rng.integers(-3000, 3001, oc).astype(np.int32) if has_bias else None
    sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
    kdim = kernel[0] * kernel[1] * (1 if dw else ic)
    so = float(sx * sw.mean() * np.sqrt(kdim) * 60)
    zo = int(rng.integers(-20, 21))
    return dict(x=x, w=w, bias=bias, shape=shape, sx=sx, zx=zx, sw=sw, zw=zw, so=so, zo=zo, act=act)


@pytest.mark.parametrize("idx", range(len(CONV_CASES)))
def test_conv_closed_form_and_nnacl(orc, idx):
    from oracle import pyoracle
    have_ref = pyoracle.Reference.available()
    rng = np.random.default_rng(100 + idx)
    for it in range(6):
        case = _conv_case(rng, *CONV_CASES[idx], bool(it & 1), bool(it & 2), it != 3, [0, 1, 3][it % 3])
        got = orc.conv_int8(**case)
        want = cf.conv_int8(case["x"], case["w"], case["bias"], case["shape"], case["sx"], case["zx"], case["sw"],
                            case["zw"], case["so"], case["zo"], case["act"])
        assert np.array_equal(got, want), (idx, it)
        if have_ref:
            r = pyoracle.reference()
            r.threads = 1 + it % 3
            assert np.array_equal(got, r.conv_int8(**case)), (idx, it)


@pytest.mark.parametrize("geom", [(1, 6, 7, 3, 5), (2, 9, 8, 16, 12), (1, 14, 14, 32, 24), (1, 3, 3, 1, 1)])
def test_dense_3x3_stride_1_is_conv_int8_when_the_reference_selects_it(orc, geom):
    """Dense 3x3 stride-1 convolutions: the reference runs ConvInt8 on them on ARM64 cores with dot product and a
    Winograd kernel elsewhere (convolution_int8_creator.cc:81-94).  The oracle restates ConvInt8; it is checked here
    against the closed form and against the compiled ConvInt8 itself, reached without the x86 kernel selection."""
    from oracle import pyoracle
    b, ih, iw, ic, oc = geom
    rng = np.random.default_rng(500 + ih + ic)
    for it in range(6):
        pad = [(1, 1, 1, 1), (0, 0, 0, 0), (2, 1, 0, 2)][it % 3]
        if ih + pad[0] + pad[1] < 3 or iw + pad[2] + pad[3] < 3:
            continue
        case = _conv_case(rng, b, ih, iw, ic, oc, (3, 3), (1, 1), (1, 1), pad, bool(it & 1), bool(it & 2), it != 3,
                          [0, 1, 3][it % 3])
        got = orc.conv_int8_as_arm64_sdot(**case)
        want = cf.conv_int8(case["x"], case["w"], case["bias"], case["shape"], case["sx"], case["zx"], case["sw"],
                            case["zw"], case["so"], case["zo"], case["act"])
        assert np.array_equal(got, want), (geom, it)
        if pyoracle.Reference.available():
            r = pyoracle.reference()
            r.threads = 1 + it % 3
            assert np.array_equal(got, r.conv_int8_as_arm64_sdot(**case)), (geom, it)
            with pytest.raises(RuntimeError):  # the x86 selection refuses: Winograd there
                r.conv_int8(**case)


def test_conv1x1_input_pack_reference_vectors(orc):
    """Input1x1PrePack1/2 of the reference (mindspore/lite/test/ut/src/runtime/kernel/arm/int8/
    conv_1x1_int8_tests.cc:32-71) pin the strided/padded 1x1 gather with its zero fill.  With an identity 1x1
    weight, zero zero-points and a real multiplier of exactly 1, the convolution output IS the gathered buffer, so
    the oracle's conv must reproduce the `correct` vectors of those tests (same in/out geometry as the tests set)."""
    from oracle.pyoracle import ConvShape
    in1 = np.array([4, 13, -3, 16, 19, 8, 19, -6, -2, -9, 9, 18, 23, 8, 47, -14, 15, 4, -0, 37, -0, 6, 0, -1, 37, 13,
                    11, 1, -1, 41, 9, 14, 3, 0, 8, 9, 14, -14, -8, -8, -8, 7, 19, 17, 13, 3, 9, 18, -1, -0, 18, 0, 4,
                    -2], np.int8).reshape(1, 3, 3, 6)
    correct1 = np.array([0] * 24 + [37, 13, 11, 1, -1, 41] + [0] * 24, np.int8)
    shape1 = ConvShape(1, 3, 3, 6, 3, 3, 6, 1, 1, 2, 2, 1, 1, 1, 1)
    out1 = orc.conv_int8(in1, np.eye(6, dtype=np.int8).reshape(6, 1, 1, 6), None, shape1, 1.0, 0, [1.0], [0], 1.0, 0)
    assert np.array_equal(out1.reshape(-1), correct1)

    in2 = np.array([-0, -0, -7, -0, -6, 4, 9, 9, 12, -0, 6, 2, 13, 15, 16, -7, 9, 1, 10, 13, 17, 17, 4, 13, -6, 5, 7,
                    -7, 15, 0, 1, -5, -7, 18, 15, 19, -7, 13, 7, -0, 16, -5, 16, -7, 6, 10, -5, 10, 9, 12, -9, -8, -4,
                    18, -5, 0, 7, 12, 13, 16, -9, -4, 18, -0, 8, 6, 2, 10, 16, 1, -1, 2, 9, 8, 9, 13, 7, -0, 15, -7, 0,
                    -0, 17, 19, 9, 17, -6, -2, 7, -0, 10, -6, -6, 18, -0, 9, 9, 6, 3, -1, -8, 10, 17, -9, 17, 6, -3, 7,
                    -2, -0, -9, 1, -3, 15, 13, 4, 18], np.int8).reshape(1, 9, 13, 1)
    correct2 = np.array([0, 0, 0, 0, 0, 0, 15, -7, -7, 0, 0, 0, 9, 7, 0, 0, 0, 0, 0, 0], np.int8)
    shape2 = ConvShape(1, 9, 13, 1, 4, 5, 1, 1, 1, 4, 4, 1, 1, 2, 2)
    out2 = orc.conv_int8(in2, np.ones((1, 1, 1, 1), np.int8), None, shape2, 1.0, 0, [1.0], [0], 1.0, 0)
    assert np.array_equal(out2.reshape(-1), correct2)


DW_CASES = [
    (1, 6, 6, 5, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (2, 7, 5, 8, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1)),
    (1, 9, 9, 3, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2)),
    (1, 5, 8, 16, (5, 5), (1, 2), (1, 1), (2, 2, 2, 2)),
]


@pytest.mark.parametrize("idx", range(len(DW_CASES)))
def test_depthwise_closed_form_and_nnacl(orc, idx):
    from oracle import pyoracle
    have_ref = pyoracle.Reference.available()
    rng = np.random.default_rng(200 + idx)
    b, ih, iw, ch, kernel, stride, dil, pad = DW_CASES[idx]
    for it in range(6):
        case = _conv_case(rng, b, ih, iw, ch, ch, kernel, stride, dil, pad, bool(it & 1), bool(it & 2), it != 3,
                          [0, 1, 3][it % 3], dw=True)
        got = orc.conv_dw_int8(**case)
        want = cf.conv_int8(case["x"], case["w"], case["bias"], case["shape"], case["sx"], case["zx"], case["sw"],
                            case["zw"], case["so"], case["zo"], case["act"], depthwise=True)
        assert np.array_equal(got, want), (idx, it)
        if have_ref:
            r = pyoracle.reference()
            r.threads = 1 + it % 3
            assert np.array_equal(got, r.conv_dw_int8(**case)), (idx, it)


def _dq_inputs():
    rng = np.random.default_rng(300)
    xs = [rng.standard_normal(5000).astype(np.float32), rng.standard_normal((37, 91)).astype(np.float32) * 5 + 3,
          np.zeros(700, np.float32), np.full(1000, 2.5, np.float32), np.array([1.0], np.float32),
          rng.uniform(-1e-3, 1e-3, 4096).astype(np.float32), np.linspace(-7.5, 9.25, 3001, dtype=np.float32),
          (rng.standard_normal(2048) * 1e6).astype(np.float32)]
    sp = rng.standard_normal(3000).astype(np.float32)
    sp[5], sp[77], sp[900] = np.nan, 12.5, -13.25
    xs.append(sp)
    return xs


def test_dynamic_quant_closed_form(orc):
    for x in _dq_inputs():
        for sym in (False, True):
            q, scale, zp = orc.dynamic_quant(x, sym)
            s2, z2 = cf.dynquant_params(x, sym)
            assert (scale, zp) == (s2, z2)
            assert np.array_equal(q, cf.quantize_fp32_int8(x, np.float32(scale), zp))


def test_quantize_special_values(orc, ref):
    x = np.array([np.inf, -np.inf, np.nan, 3e38, -3e38, 0.0, -0.0, 0.5, -0.5, 1.5, 2.5, -2.5, 126.5, 127.5, -128.5,
                  -129.0, 1e10, -1e10, 2147483520.0, 4e9], np.float32)
    for scale, zp in [(1.0, 0), (0.5, 3), (0.0371, -128), (1e-30, 0), (3.0, 127)]:
        got = orc.quantize_fp32_int8(x, scale, zp)
        assert np.array_equal(got, cf.quantize_fp32_int8(x, scale, zp)), (scale, zp)
        assert np.array_equal(got, ref.quantize_fp32_int8(x, scale, zp)), (scale, zp)


def test_quantize_hand_computed(orc):
    """Hand-computed answers: scale 0.5 (inverse exactly 2), zp 3 -> q = round_half_away(2x + 3)."""
    x = np.array([0.25, -0.25, 1.0, -1.75, -2.25, 61.75, 62.0, 100.0, -65.25, -65.5, -66.0, -200.0], np.float32)
    #            3.5    2.5    5    -0.5   -1.5   126.5  127   203    -127.5  -128   -129   -397
    want = [4, 3, 5, -1, -2, 127, 127, 127, -128, -128, -128, -128]
    assert orc.quantize_fp32_int8(x, 0.5, 3).tolist() == want


def test_dynamic_quant_vs_nnacl(orc, ref):
    for i, x in enumerate(_dq_inputs()):
        for sym in (False, True):
            ref.threads = 1 + i % 4
            q, s, z = orc.dynamic_quant(x, sym)
            q2, s2, z2 = ref.dynamic_quant(x, sym)
            assert (s, z) == (s2, z2)
            assert np.array_equal(q, q2)


def test_dynamic_quant_segments_closed_form_and_nnacl(orc, ref):
    """One {scale, zero point} per contiguous run: every run must equal the per-tensor closed form applied to that run
    alone (a mistake in the run boundaries or a shared min/max fails), and the compiled nnacl sequence."""
    rng = np.random.default_rng(310)
    for segments, unit in [(1, 50), (7, 1), (37, 91), (16, 768), (3, 5000)]:
        x = (rng.standard_normal((segments, unit)) * rng.uniform(0.1, 20, (segments, 1))).astype(np.float32)
        if segments > 2 and unit > 1:
            x[1] = -3.5                 # constant run
            x[2, unit // 2] = np.nan    # never selected (a run of nothing but NaN is outside the closed form)
        for sym in (False, True):
            q, scales, zps = orc.dynamic_quant_segments(x, sym)
            for i in range(segments):
                s2, z2 = cf.dynquant_params(x[i], sym)
                assert (scales[i], zps[i]) == (s2, z2), (segments, unit, i)
                assert np.array_equal(q[i], cf.quantize_fp32_int8(x[i], np.float32(scales[i]), int(zps[i])))
            q2, sc2, zp2 = ref.dynamic_quant_segments(x, sym)
            assert np.array_equal(q, q2) and np.array_equal(scales, sc2) and np.array_equal(zps, zp2)


def test_dynamic_matmul_rows_closed_form_and_nnacl(orc, ref):
    """Per-row input scales: row r of the result equals the per-tensor closed form evaluated with that row's scale
    (so using scale[0] everywhere, or indexing by column, fails); one input zero point for all rows."""
    rng = np.random.default_rng(410)
    for it in range(24):
        m, n, k = int(rng.integers(1, 30)), int(rng.integers(1, 30)), int(rng.integers(1, 100))
        case, w_nk = _dm_case(rng, m, n, k, bool(it & 1), 0 if it & 2 else int(rng.integers(-5, 6)), bool(it & 4),
                              [0, 1, 3][it % 3], bool(it & 8))
        sx_rows = rng.uniform(0.01, 0.1, m).astype(np.float32)
        zx = case["zx"] if it & 16 else 0
        got = orc.dynamic_matmul_rows(case["a"], case["w"], case["bias"], sx_rows, zx, case["sw"], case["zw"],
                                      case["act"], case["b_transpose"])
        for r in range(m):
            want = cf.dynamic_matmul(case["a"][r:r + 1], w_nk, case["bias"], sx_rows[r], zx, case["sw"],
                                     int(case["zw"][0]), case["act"])
            assert np.array_equal(got[r:r + 1].view(np.uint32), want.view(np.uint32)), (it, r)
        ref.threads = 1 + it % 3
        got2 = ref.dynamic_matmul_rows(case["a"], case["w"], case["bias"], sx_rows, zx, case["sw"], case["zw"],
                                       case["act"], case["b_transpose"])
        assert np.array_equal(got.view(np.uint32), got2.view(np.uint32)), it


def test_minmax(orc, ref):
    rng = np.random.default_rng(301)
    x = rng.standard_normal(10007).astype(np.float32)
    x[3] = np.nan
    assert orc.minmax(x) == ref.minmax(x) == (float(np.nanmin(x)), float(np.nanmax(x)))
    e = np.empty(0, np.float32)
    assert orc.minmax(e) == (float(np.finfo(np.float32).max), -float(np.finfo(np.float32).max))


def _dm_case(rng, m, n, k, peroc, zw0, has_bias, act, bt=True):
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w_nk = rng.integers(-128, 128, (n, k), dtype=np.int8)
    nf = n if peroc else 1
    sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
    zw = np.full(nf, zw0, np.int32)
    bias = rng.standard_normal(n).astype(np.float32) if has_bias else None
    w = w_nk if bt else np.ascontiguousarray(w_nk.T)
    return dict(a=a, w=w, bias=bias, sx=float(rng.uniform(0.01, 0.1)), zx=int(rng.integers(-128, 128)), sw=sw, zw=zw,
                act=act, b_transpose=bt), w_nk


def test_dynamic_matmul_closed_form_and_nnacl(orc):
    from oracle import pyoracle
    have_ref = pyoracle.Reference.available()
    rng = np.random.default_rng(400)
    for it in range(48):
        m, n, k = int(rng.integers(1, 30)), int(rng.integers(1, 30)), int(rng.integers(1, 100))
        case, w_nk = _dm_case(rng, m, n, k, bool(it & 1), 0 if it & 2 else int(rng.integers(-5, 6)), bool(it & 4),
                              [0, 1, 3][it % 3], bool(it & 8))
        got = orc.dynamic_matmul(**case)
        want = cf.dynamic_matmul(case["a"], w_nk, case["bias"], case["sx"], case["zx"], case["sw"],
                                 int(case["zw"][0]), case["act"])
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), it
        if have_ref:
            r = pyoracle.reference()
            r.threads = 1 + it % 3
            assert np.array_equal(got.view(np.uint32), r.dynamic_matmul(**case).view(np.uint32)), it
