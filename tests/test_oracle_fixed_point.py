"""Pins the oracle's fixed-point and quant-parameter functions against exact integer / rational closed forms and,
where it is built, against the compiled nnacl (NN/int8/fixed_point.c, NN/int8/quantize.c)."""
import math
import random
import struct

import numpy as np
import pytest

from tests import closed_forms as cf

EDGE = [0, 1, -1, 2, -2, 3, -3, 127, -128, (1 << 30), -(1 << 30), (1 << 30) + 1, -(1 << 30) - 1, (1 << 30) - 1,
        cf.INT32_MAX, cf.INT32_MIN, cf.INT32_MAX - 1, cf.INT32_MIN + 1, 0x40000000, 0x7FFFFF80, 12345678, -87654321]


def test_srdhm_edges_and_random(orc):
    rnd = random.Random(1)
    pairs = [(a, b) for a in EDGE for b in EDGE]
    pairs += [(rnd.randint(cf.INT32_MIN, cf.INT32_MAX), rnd.randint(cf.INT32_MIN, cf.INT32_MAX)) for _ in range(30000)]
    # products that land exactly on a rounding tie: a*b + 2^30 == k * 2^31  <=>  a*b == 2^30 (mod 2^31)
    pairs += [(1 << 30, 2 * j + 1) for j in range(-50, 50)] + [(-(1 << 30), 2 * j + 1) for j in range(-50, 50)]
    pairs += [(1 << 15, (2 * j + 1) << 15) for j in range(-50, 50)]
    for a, b in pairs:
        assert orc.srdhm(a, b) == cf.srdhm(a, b), (a, b)


def test_srdhm_tie_direction(orc):
    # -0.5 -> 0 and +0.5 -> 1: ties go toward +infinity, not away from zero
    assert orc.srdhm(1 << 30, 1) == 1
    assert orc.srdhm(-(1 << 30), 1) == 0
    assert orc.srdhm(-(1 << 30), 3) == -1  # -1.5 -> -1
    assert orc.srdhm(cf.INT32_MIN, cf.INT32_MIN) == cf.INT32_MAX


def test_rdiv_pot(orc):
    rnd = random.Random(2)
    xs = EDGE + [rnd.randint(cf.INT32_MIN, cf.INT32_MAX) for _ in range(3000)]
    for e in list(range(0, 33)) + [40, -1]:
        half = 1 << max(e - 1, 0)
        for x in xs + [half, -half, 3 * half, -3 * half, half - 1, -half + 1, half + 1, -half - 1]:
            if not cf.INT32_MIN <= x <= cf.INT32_MAX:
                continue
            assert orc.rdiv_pot(x, e) == cf.rdiv_pot(x, e), (x, e)
    assert orc.rdiv_pot(3, 1) == 2 and orc.rdiv_pot(-3, 1) == -2  # +-1.5 -> +-2: ties away from zero
    assert orc.rdiv_pot(1, 1) == 1 and orc.rdiv_pot(-1, 1) == -1


def test_mul_by_quant_mult(orc):
    rnd = random.Random(3)
    for _ in range(30000):
        v = rnd.randint(cf.INT32_MIN, cf.INT32_MAX) if rnd.random() < 0.3 else rnd.randint(-(1 << 22), 1 << 22)
        mult = rnd.randint(1 << 30, cf.INT32_MAX) * rnd.choice([1, 1, 1, -1])
        if rnd.random() < 0.7:
            ls, rs = 0, -rnd.randint(0, 31)
        else:
            ls, rs = rnd.randint(0, 8), 0
        assert orc.mul_by_quant_mult(v, mult, ls, rs) == cf.mbqm(v, mult, ls, rs), (v, mult, ls, rs)


def _doubles():
    rnd = random.Random(4)
    vals = [0.0, -0.0, 1.0, -1.0, 0.5, 0.25, 0.75, 1.5, 2.0, 3.0, 1e-3, 1e-9, 1e9, 1e300, 1e-300, 5e-324, 2.2e-308,
            1.1e-308, math.inf, -math.inf, math.nan, 0.9999999999999999, 0.99999999976716936,  # carry case
            float.fromhex("0x1.fffffffffffffp-1"), float.fromhex("0x1.fffffffcp-1"), float.fromhex("0x1.fffffffep-1"),
            float.fromhex("0x1.00000001p-3"), float.fromhex("0x1.000000008p-3"), float.fromhex("0x1.000000018p-3")]
    for _ in range(15000):
        bits = rnd.getrandbits(64)
        vals.append(struct.unpack("<d", struct.pack("<Q", bits))[0])
    for _ in range(15000):
        vals.append(rnd.uniform(1e-6, 4.0) * rnd.choice([1, -1]))
    return vals


def test_quantize_multiplier_exact(orc):
    for m in _doubles():
        assert orc.quantize_multiplier(m) == cf.quantize_multiplier(m), m.hex() if not math.isnan(m) else m
        assert orc.round_param(m) == cf.round_param(m)


def test_round_param_single_known_answers(orc):
    """Hand-computed: the mantissa field is the low 23 bits of trunc(m), the exponent field the bits above."""
    assert orc.round_param_single(0.0) == (0x40000000, 0, -126)
    assert orc.round_param_single(0.75) == (0x40000000, 0, -126)       # any multiplier below 1 truncates to 0
    assert orc.round_param_single(1.0) == (0x40000080, 0, -126)        # mantissa field 1
    assert orc.round_param_single(8388607.9) == (0x7FFFFF80, 0, -126)  # mantissa field all ones
    assert orc.round_param_single(8388608.0) == (0x40000000, 0, -125)  # 2^23: exponent field 1
    assert orc.round_param_single(126.0 * 8388608.0) == (0x40000000, 0, 0)
    assert orc.round_param_single(127.0 * 8388608.0 + 3.0) == (0x40000180, 1, 0)
    rnd = random.Random(4)
    for _ in range(20000):
        m = rnd.uniform(0.0, 2.0 ** 32 - 1.0)
        assert orc.round_param_single(m) == cf.round_param_single(m), m


def test_round_param_single_vs_nnacl(orc, ref):
    rnd = random.Random(5)
    for m in [0.0, 0.3, 1.0, 8388608.0, 4294967295.0] + [rnd.uniform(0.0, 2.0 ** 32 - 1.0) for _ in range(20000)]:
        assert orc.round_param_single(m) == ref.round_param_single(m), m


def test_quantize_multiplier_value(orc):
    # mult * 2^(shift-31) reproduces m to 31 bits
    for m in [0.0003, 0.02 * 0.005 / 0.05, 0.7, 1.0, 123.456]:
        mult, shift = orc.quantize_multiplier(m)
        assert (1 << 30) <= mult < (1 << 31)
        assert abs(mult * 2.0 ** (shift - 31) - m) <= m * 2.0 ** -31


def test_act_range(orc):
    rnd = random.Random(5)
    for _ in range(5000):
        zp = rnd.randint(-128, 127)
        scale = float(np.float32(rnd.uniform(1e-3, 0.5)))
        for relu, relu6 in [(0, 0), (1, 0), (0, 1)]:
            assert orc.act_range(relu, relu6, zp, scale) == cf.act_range(relu, relu6, zp, scale)
    assert orc.act_range(0, 1, -128, 6.0 / 255.0) in [(-128, 127)]
    assert orc.act_range(1, 0, 5, 0.05) == (5, 127)


def test_requant_params(orc):
    rnd = np.random.default_rng(6)
    sw = rnd.uniform(1e-4, 1e-2, 4096)
    for sx, so in [(0.02, 0.05), (0.0123456789, 0.3), (1.0, 1e-4)]:
        got = orc.requant_params(sx, sw, so)
        want = cf.requant_params(sx, sw, so)
        for g, w in zip(got, want):
            assert np.array_equal(g.astype(np.int64), w)


# ---------------------------------------------------------------- against the compiled nnacl
def test_fixed_point_vs_nnacl(orc, ref):
    rnd = random.Random(7)
    for a in EDGE:
        for b in EDGE:
            assert orc.srdhm(a, b) == ref.srdhm(a, b), (a, b)
    for _ in range(30000):
        a, b = rnd.randint(cf.INT32_MIN, cf.INT32_MAX), rnd.randint(cf.INT32_MIN, cf.INT32_MAX)
        assert orc.srdhm(a, b) == ref.srdhm(a, b)
        e = rnd.randint(0, 31)
        assert orc.rdiv_pot(a, e) == ref.rdiv_pot(a, e)
        mult = rnd.randint(1 << 30, cf.INT32_MAX)
        ls, rs = (0, -e) if rnd.random() < 0.7 else (rnd.randint(0, 8), 0)
        assert orc.mul_by_quant_mult(a, mult, ls, rs) == ref.mul_by_quant_mult(a, mult, ls, rs)


def test_quantize_multiplier_vs_nnacl(orc, ref):
    for m in _doubles():
        assert orc.quantize_multiplier(m) == ref.quantize_multiplier(m), m
        assert orc.round_param(m) == ref.round_param(m), m


def test_act_range_vs_nnacl(orc, ref):
    rnd = random.Random(8)
    for _ in range(5000):
        zp = rnd.randint(-128, 127)
        scale = float(np.float32(rnd.uniform(1e-3, 0.5)))
        for relu, relu6 in [(0, 0), (1, 0), (0, 1)]:
            assert orc.act_range(relu, relu6, zp, scale) == ref.act_range(bool(relu), bool(relu6), zp, scale)
