"""Randomised differential parity: the GPU library against the CPU oracle over seeded random shapes, layouts and quant
parameters (row counts on both sides of every kernel switch, ragged K and N, per-tensor and per-channel weights with
and without zero points, every activation).  Every case is a full-tensor, bit-exact comparison."""
import numpy as np
import pytest

from mindspore_amd import kernels as K
from tests import test_gpu_parity as T

pytestmark = pytest.mark.gpu

M_EDGES = [1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 64, 65, 127, 128, 129, 200, 257, 511, 700]
N_EDGES = [1, 3, 4, 16, 64, 100, 128, 192, 255, 256, 257, 512, 768, 1000]
K_EDGES = [1, 15, 16, 17, 63, 64, 65, 128, 255, 256, 768, 1000, 1024, 1040, 2048, 3000, 4096]


def _pick(rng, choices):
    return choices[int(rng.integers(0, len(choices)))]


def _flag(rng):
    return bool(rng.integers(0, 2))


@pytest.mark.parametrize("seed", [1, 2])
def test_random_matmul(orc, seed):
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    for it in range(500):
        m = _pick(rng, M_EDGES) if rng.random() < 0.6 else int(rng.integers(1, 400))
        n = _pick(rng, N_EDGES) if rng.random() < 0.6 else int(rng.integers(1, 900))
        k = _pick(rng, K_EDGES) if rng.random() < 0.6 else int(rng.integers(1, 2500))
        case = T._mm_case(rng, m, n, k, _flag(rng), _flag(rng), _flag(rng), _pick(rng, [0, 1, 3]), _flag(rng))
        got, _ = T._gpu_matmul(case, device_tensors=_flag(rng))
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (seed, it, m, n, k, int((got != want).sum()))


@pytest.mark.parametrize("seed", [5])
def test_random_few_tiles_long_k(orc, seed):
    """A few hundred rows against a reduction of 1024 bytes and more: the 64 x 64 and 64-channel x 128-row tiles on eight
    stages that such shapes take while they fit the device in one round, and their neighbours (the K-block tiles
    beyond); handles with and without the blocked weight copy; int8 and fp32 output."""
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    for it in range(40):
        m = int(rng.integers(129, 1200))
        n = _pick(rng, [64, 100, 256, 500, 768, 1000, 2048, 4100]) if rng.random() < 0.5 else int(rng.integers(4, 3000))
        k = _pick(rng, [1024, 1040, 2048, 2064, 3072, 4096, 4112]) if rng.random() < 0.6 else int(rng.integers(1009, 4600))
        if m * n * k > 4e9:
            m = max(129, int(4e9 / (n * k)))
        if it % 4 != 3:
            case = T._mm_case(rng, m, n, k, _flag(rng), _flag(rng), _flag(rng), _pick(rng, [0, 1, 3]), _flag(rng))
            got, _ = T._gpu_matmul(case, device_tensors=_flag(rng), decode_pack=_flag(rng))
            want = orc.matmul_int8(**case)
            assert np.array_equal(got, want), (seed, it, m, n, k, int((got != want).sum()))
        else:
            a = rng.integers(-128, 128, (m, k), dtype=np.int8)
            w = rng.integers(-128, 128, (n, k), dtype=np.int8)
            nf = n if _flag(rng) else 1
            sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
            zw = np.full(nf, 0 if _flag(rng) else int(rng.integers(-5, 6)), np.int32)
            bias = rng.standard_normal(n).astype(np.float32) if _flag(rng) else None
            sx, zx, act = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128)), _pick(rng, [0, 1, 3])
            kern = K.MatmulDynamicInt8Kernel(w, bias, T._qps(sw, zw), True, act)
            want = orc.dynamic_matmul(a, w, bias, sx, zx, sw, zw, act, True)
            got = kern.run(a, K.QuantParam(sx, zx))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (seed, it, m, n, k)


@pytest.mark.parametrize("seed", [11])
def test_random_decode_rows_against_wide_matrices(orc, seed):
    """2..32 activation rows against 8192 channels and more with K up to 4096: the matrix-core decode kernel with three
    channel groups per workgroup (ragged last workgroups, ragged K, zero points, every activation), singly and as a
    group launch of two members."""
    import torch
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    for it in range(36):
        m = int(rng.integers(2, 33))
        n = _pick(rng, [8192, 8193, 8200, 8250, 9001, 11008, 12288]) if it % 3 else int(rng.integers(8192, 9400))
        k = _pick(rng, [64, 80, 1000, 1024, 2048, 3000, 4096]) if it % 2 else int(rng.integers(16, 4097))
        case = T._mm_case(rng, m, n, k, _flag(rng), _flag(rng), True, _pick(rng, [0, 1, 3]), _flag(rng))
        got, kern = T._gpu_matmul(case, device_tensors=True)
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (seed, it, m, n, k, int((got != want).sum()))
        if it % 4 == 0:  # the same handle and a narrower one as one launch
            c2 = T._mm_case(rng, m, int(rng.integers(16, 600)), k, True, _flag(rng), True, 0)
            c2.update(a=case["a"], sx=case["sx"], zx=case["zx"])
            k2 = K.MatmulInt8Kernel(c2["w"], c2["bias"], K.QuantParam(c2["sx"], c2["zx"]), T._qps(c2["sw"], c2["zw"]),
                                    K.QuantParam(c2["so"], c2["zo"]), c2["b_transpose"], c2["act"])
            outs = K.matmul_run_group([kern, k2], torch.from_numpy(case["a"]).cuda())
            torch.cuda.synchronize()
            assert np.array_equal(outs[0].cpu().numpy(), want), (seed, it, "group member 0")
            assert np.array_equal(outs[1].cpu().numpy(), orc.matmul_int8(**c2)), (seed, it, "group member 1")


@pytest.mark.parametrize("seed", [3])
def test_random_dynamic_matmul(orc, seed):
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    for it in range(300):
        m, n, k = int(rng.integers(1, 300)), int(rng.integers(1, 500)), int(rng.integers(1, 1500))
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        w = rng.integers(-128, 128, (n, k), dtype=np.int8)
        nf = n if _flag(rng) else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = np.full(nf, 0 if _flag(rng) else int(rng.integers(-5, 6)), np.int32)
        bias = rng.standard_normal(n).astype(np.float32) if _flag(rng) else None
        sx, zx, act = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128)), _pick(rng, [0, 1, 3])
        kern = K.MatmulDynamicInt8Kernel(w, bias, T._qps(sw, zw), True, act)
        want = orc.dynamic_matmul(a, w, bias, sx, zx, sw, zw, act, True)
        got = kern.run(a, K.QuantParam(sx, zx))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (seed, it, m, n, k)


def _geometry(rng):
    kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    pad = tuple(int(rng.integers(0, 3)) for _ in range(4))
    return kh, kw, stride, dil, pad


@pytest.mark.parametrize("seed", [4])
def test_random_conv(orc, seed):
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    ran = 0
    for it in range(400):
        b, ih, iw = int(rng.integers(1, 3)), int(rng.integers(1, 20)), int(rng.integers(1, 20))
        ic, oc = _pick(rng, [1, 3, 4, 7, 16, 17, 32]), _pick(rng, [1, 3, 4, 8, 17, 32, 65, 64, 100, 128])
        kh, kw, stride, dil, pad = _geometry(rng)
        if ih + pad[0] + pad[1] < (kh - 1) * dil[0] + 1 or iw + pad[2] + pad[3] < (kw - 1) * dil[1] + 1:
            continue
        case = T._conv_case(rng, b, ih, iw, ic, oc, (kh, kw), stride, dil, pad, _flag(rng), _flag(rng), _flag(rng),
                            _pick(rng, [0, 1, 3]))
        try:
            got = T._gpu_conv(case, stride, dil, pad, 1, device_tensors=_flag(rng))
        except K._lib.MiError as e:
            # dense 3x3 stride-1 dilation-1 is declined: the x86 reference runs an integer Winograd there
            assert e.code == K._lib.MI_NOT_SUPPORT and (kh, kw, stride, dil) == (3, 3, (1, 1), (1, 1)), (it, e)
            continue
        want = orc.conv_int8(**case)
        ran += 1
        assert np.array_equal(got, want), (seed, it, b, ih, iw, ic, oc, kh, kw, stride, dil, pad)
    assert ran > 250


@pytest.mark.parametrize("seed", [5])
def test_random_depthwise(orc, seed):
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    ran = 0
    for it in range(300):
        b, ih, iw = int(rng.integers(1, 3)), int(rng.integers(1, 24)), int(rng.integers(1, 24))
        c = _pick(rng, [2, 3, 8, 16, 24, 32, 48])
        kh, kw, stride, dil, pad = _geometry(rng)
        if ih + pad[0] + pad[1] < (kh - 1) * dil[0] + 1 or iw + pad[2] + pad[3] < (kw - 1) * dil[1] + 1:
            continue
        case = T._conv_case(rng, b, ih, iw, c, c, (kh, kw), stride, dil, pad, _flag(rng), _flag(rng), _flag(rng),
                            _pick(rng, [0, 1, 3]), dw=True)
        got = T._gpu_conv(case, stride, dil, pad, c, device_tensors=_flag(rng))
        ran += 1
        assert np.array_equal(got, orc.conv_dw_int8(**case)), (seed, it, b, ih, iw, c, kh, kw, stride, dil, pad)
    assert ran > 200


@pytest.mark.parametrize("seed", [6])
def test_random_matmul_large_tiles(orc, seed):
    """Shapes large enough for every tile configuration of the GEMM (64, 128 with two and three workgroups per CU,
    256 x 128, 256 x 256), int8 and fp32 epilogues, random flags."""
    rng = np.random.default_rng(seed)
    orc.set_threads(16)
    shapes = [(2100, 1300, 48), (2048 + 37, 2048 + 4, 272), (4224, 2100, 144), (4100, 2700, 1040), (4096, 3100, 80),
              (4500, 3600, 16), (300, 11008, 80), (512, 8200, 272), (700, 640, 3000), (1500, 1500, 1024)]
    for it, (m, n, k) in enumerate(shapes):
        case = T._mm_case(rng, m, n, k, _flag(rng), _flag(rng), _flag(rng), _pick(rng, [0, 1, 3]), _flag(rng))
        got, _ = T._gpu_matmul(case, device_tensors=True)
        want = orc.matmul_int8(**case)
        assert np.array_equal(got, want), (seed, it, m, n, k, int((got != want).sum()))
        # the same operands through the fp32 (dynamic MatMul) epilogue
        w_nk = case["w"] if case["b_transpose"] else np.ascontiguousarray(case["w"].T)
        sw, zw = case["sw"], case["zw"]
        if len(zw) > 1:
            zw = np.zeros_like(zw)  # per-channel dynamic weights are symmetric in the reference
        bias = rng.standard_normal(n).astype(np.float32) if _flag(rng) else None
        act = _pick(rng, [0, 1, 3])
        kern = K.MatmulDynamicInt8Kernel(w_nk, bias, T._qps(sw, zw), True, act)
        wantf = orc.dynamic_matmul(case["a"], w_nk, bias, 0.037, case["zx"], sw, zw, act, True)
        gotf = kern.run(case["a"], K.QuantParam(0.037, case["zx"]))
        assert np.array_equal(gotf.view(np.uint32), wantf.view(np.uint32)), (seed, it, m, n, k, "fp32")
