"""Seeded synthetic inputs for the five benchmark configurations of the int8 hot path.

Random numbers come from a counter-based SplitMix64 stream implemented with NumPy integer arithmetic only, so the
same (seed, stream) pair yields the same bytes on every machine and NumPy build; the normal variates use a
Box-Muller transform in float64.
"""
import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(counter):
    with np.errstate(over="ignore"):
        z = counter + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


class Stream:
    """Independent random stream keyed by (seed, stream id)."""

    def __init__(self, seed, stream):
        key = _splitmix64(np.array([seed], np.uint64))[0] ^ _splitmix64(np.array([stream + 0x51ED27], np.uint64))[0]
        self._base = np.uint64(key)
        self._pos = 0

    def bits(self, n):
        with np.errstate(over="ignore"):
            ctr = self._base + (np.arange(self._pos, self._pos + n, dtype=np.uint64) * np.uint64(0x2545F4914F6CDD1D))
        self._pos += n
        return _splitmix64(ctr)

    def integers(self, lo, hi, shape):
        """Uniform integers in [lo, hi] inclusive."""
        n = int(np.prod(shape))
        span = np.uint64(hi - lo + 1)
        return ((self.bits(n) >> np.uint64(11)) % span).astype(np.int64).reshape(shape) + lo

    def uniform(self, lo, hi, shape):
        n = int(np.prod(shape))
        u = (self.bits(n) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        return (lo + (hi - lo) * u).reshape(shape)

    def normal(self, shape):
        n = int(np.prod(shape))
        half = (n + 1) // 2
        u1 = ((self.bits(half) >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (self.bits(half) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        r = np.sqrt(-2.0 * np.log(u1))
        z = np.concatenate([r * np.cos(2.0 * np.pi * u2), r * np.sin(2.0 * np.pi * u2)])[:n]
        return z.reshape(shape)


def fc_c1(seed=0):
    """Config 1: FullConnection 128x768 -> 768, per-channel symmetric weights, int32 bias."""
    s = Stream(seed, 1)
    m, k, n = 128, 768, 768
    return dict(
        a=s.integers(-128, 127, (m, k)).astype(np.int8), w=s.integers(-128, 127, (n, k)).astype(np.int8),
        bias=s.integers(-5000, 5000, (n,)).astype(np.int32), sx=0.02, zx=-3,
        sw=s.uniform(0.001, 0.01, (n,)).astype(np.float32).astype(np.float64), zw=np.zeros(n, np.int32), so=0.05,
        zo=5, act=0)


def gemm_c5(size, seed=0):
    """Config 5: square int8 GEMM M=N=K=size with per-channel requantisation."""
    s = Stream(seed, 500 + size)
    m = n = k = size
    sw = s.uniform(1e-4, 1e-2, (n,)).astype(np.float32).astype(np.float64)
    sx = 0.02
    so = float(np.float32(sx * float(np.mean(sw)) * np.sqrt(k) * 150.0))
    return dict(
        a=s.integers(-128, 127, (m, k)).astype(np.int8), w=s.integers(-128, 127, (n, k)).astype(np.int8),
        bias=s.integers(-5000, 5000, (n,)).astype(np.int32), sx=sx, zx=7, sw=sw, zw=np.zeros(n, np.int32), so=so,
        zo=0, act=0)


DECODE_SHAPES = [("qkv", 12288, 4096), ("o", 4096, 4096), ("gate", 11008, 4096), ("up", 11008, 4096),
                 ("down", 4096, 11008)]


def gemv_c4(name, n, k, m, seed=0):
    """Config 4: decode GEMV, activation [m,k], weights clip(round(N(0,1)*32), +-127) per-channel symmetric."""
    s = Stream(seed, 400 + sum(map(ord, name)) + 7 * m)
    w = np.clip(np.round(s.normal((n, k)) * 32.0), -127, 127).astype(np.int8)
    sw = s.uniform(0.001, 0.01, (n,)).astype(np.float32).astype(np.float64)
    sx = 0.05
    so = float(np.float32(sx * float(np.mean(sw)) * np.sqrt(k) * 32.0 * 2.0))
    return dict(
        a=s.integers(-128, 127, (m, k)).astype(np.int8), w=w, bias=s.integers(-5000, 5000, (n,)).astype(np.int32),
        sx=sx, zx=int(s.integers(-8, 8, (1,))[0]), sw=sw, zw=np.zeros(n, np.int32), so=so, zo=0, act=0)


BERT_SHAPES = [("qkv", 2304, 768), ("out", 768, 768), ("ffn1", 3072, 768), ("ffn2", 768, 3072)]


def bert_c3_activation(k, rows=4096, seed=0):
    """Config 3 activation: N(0,1) with 1% of the entries replaced by +-8."""
    s = Stream(seed, 300 + k)
    x = s.normal((rows, k))
    u = s.uniform(0.0, 1.0, (rows, k))
    sign = np.where(s.integers(0, 1, (rows, k)) == 0, -1.0, 1.0)
    x = np.where(u < 0.01, 8.0 * sign, x)
    return x.astype(np.float32)


def bert_c3_weights(name, n, k, seed=0):
    s = Stream(seed, 350 + sum(map(ord, name)))
    return dict(w=s.integers(-127, 127, (n, k)).astype(np.int8),
                sw=s.uniform(0.001, 0.01, (n,)).astype(np.float32).astype(np.float64), zw=np.zeros(n, np.int32),
                bias=(s.normal((n,)) * 0.1).astype(np.float32))


def mobilenet_c2(seed=0):
    """Config 2: MobileNetV2-style block on a 1x224x224x3 int8 image.

    Returns the input image and the four layers (stem 3x3 s2, 1x1 expand, 3x3 depthwise, 1x1 project); each layer's
    quant parameters are chosen so that the ReLU6 bound lands inside the int8 range."""
    s = Stream(seed, 200)
    x = s.integers(-128, 127, (1, 224, 224, 3)).astype(np.int8)
    layers = []
    spec = [  # name, kind, ic, oc, kernel, stride, pad(u,d,l,r), act
        ("stem", "conv", 3, 32, 3, 2, (0, 1, 0, 1), 3),
        ("expand", "conv", 32, 192, 1, 1, (0, 0, 0, 0), 3),
        ("dw", "dw", 192, 192, 3, 1, (1, 1, 1, 1), 3),
        ("project", "conv", 192, 32, 1, 1, (0, 0, 0, 0), 0),
    ]
    sx = 0.02
    zx = int(s.integers(-20, 20, (1,))[0])
    for name, kind, ic, oc, ksz, stride, pad, act in spec:
        if kind == "dw":
            w = s.integers(-127, 127, (oc, ksz, ksz)).astype(np.int8)
            kdim = ksz * ksz
        else:
            w = s.integers(-127, 127, (oc, ksz, ksz, ic)).astype(np.int8)
            kdim = ksz * ksz * ic
        sw = s.uniform(0.001, 0.01, (oc,)).astype(np.float32).astype(np.float64)
        bias = s.integers(-2000, 2000, (oc,)).astype(np.int32)
        zo = int(s.integers(-20, 20, (1,))[0])
        so = 6.0 / 140.0 if act == 3 else float(np.float32(sx * float(np.mean(sw)) * np.sqrt(kdim) * 74.0 * 6.0))
        layers.append(dict(name=name, kind=kind, ic=ic, oc=oc, kernel=ksz, stride=stride, pad=pad, act=act, w=w,
                           bias=bias, sx=sx, zx=zx, sw=sw, zw=np.zeros(oc, np.int32), so=so, zo=zo))
        sx, zx = so, zo
    return x, layers
