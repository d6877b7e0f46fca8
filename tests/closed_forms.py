"""Independent mathematical statements of the int8 hot-path arithmetic, used to pin the oracle.

Everything here is exact integer / rational arithmetic (Python ints, ``fractions.Fraction``) or NumPy float32
operations that are single correctly-rounded IEEE operations; none of it mirrors the control flow of the oracle.
"""
import math
from fractions import Fraction

import numpy as np

INT32_MIN, INT32_MAX = -(1 << 31), (1 << 31) - 1


def wrap32(v):
    """Two's-complement wrap of an arbitrary Python int (or int64 array) to int32."""
    if isinstance(v, np.ndarray):
        return ((v.astype(np.int64) + (1 << 31)) % (1 << 32) - (1 << 31)).astype(np.int64)
    return (v + (1 << 31)) % (1 << 32) - (1 << 31)


def srdhm(a, b):
    """floor((a*b + 2^30) / 2^31), saturating only at a == b == INT32_MIN."""
    if a == INT32_MIN and b == INT32_MIN:
        return INT32_MAX
    return (a * b + (1 << 30)) // (1 << 31)  # Python // floors


def rdiv_pot(x, e):
    """x / 2^e rounded to nearest with ties away from zero (e capped at 31, e <= 0 is the identity)."""
    e = min(e, 31)
    if e <= 0:
        return x
    q = Fraction(x, 1 << e)
    fl = math.floor(q)
    frac = q - fl
    if frac > Fraction(1, 2):
        return fl + 1
    if frac < Fraction(1, 2):
        return fl
    return fl + 1 if x > 0 else fl  # tie: away from zero (for x < 0 floor is already the farther one)


def mbqm(v, mult, ls, rs):
    return rdiv_pot(srdhm(wrap32(v * (1 << ls)), mult), -rs)


def quantize_multiplier(m):
    """(mult, shift) with |m| = q * 2^shift, q in [0.5, 1), mult = round-half-up(q * 2^31), carry renormalised."""
    if m == 0 or math.isnan(m):
        return 0, 0
    if math.isinf(m):
        return (INT32_MIN if m < 0 else INT32_MAX), 0
    f = Fraction(abs(m))  # exact value of the double
    shift = 0
    while f >= 1:
        f /= 2
        shift += 1
    while f < Fraction(1, 2):
        f *= 2
        shift -= 1
    mult = math.floor(f * (1 << 31) + Fraction(1, 2))
    if mult == (1 << 31):
        mult >>= 1
        shift += 1
    return (-mult if m < 0 else mult), shift


def round_param(m):
    mult, shift = quantize_multiplier(m)
    return (mult, 0, shift) if shift < 0 else (mult, shift, 0)


def round_param_single(m):
    """QuantizeRoundParameterWithSinglePrecision on 0 <= m < 2**32: the VALUE of m truncated to an integer plays the
    role of the float's bit pattern (23-bit mantissa field, exponent field above it)."""
    bits = int(m)  # truncation toward zero
    mult = ((bits & 0x7FFFFF) | 0x800000) << 7
    shift = -(126 - (bits >> 23))
    return (mult, 0, shift) if shift < 0 else (mult, shift, 0)


def round_half_away(x):
    """Vector round-half-away-from-zero on float64 (what C round() does)."""
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def act_range(relu, relu6, zp, scale):
    scale = np.float32(scale)
    q0 = int(round_half_away(np.float64(np.float32(0.0) / scale + np.float32(zp))))
    q6 = int(round_half_away(np.float64(np.float32(6.0) / scale + np.float32(zp))))
    lo, hi = -128, 127
    if relu:
        lo = max(lo, q0)
    elif relu6:
        lo = max(lo, q0)
        hi = min(hi, q6)
    return lo, hi


def requant_params(sx, sw, so):
    """Real multiplier: float product of the float-narrowed scales, widened, divided by the float-narrowed output
    scale in double; then the (mult, ls, rs) split."""
    out = []
    for s in np.atleast_1d(sw):
        prod = np.float32(sx) * np.float32(s)
        real = float(np.float64(prod) / np.float64(np.float32(so)))
        out.append(round_param(real))
    a = np.array(out, dtype=np.int64)
    return a[:, 0], a[:, 1], a[:, 2]


def requant_vec(acc, mult, ls, rs, zo, amin, amax):
    """Vectorised requantisation of an int64 accumulator array (values already wrapped to int32); per-column
    mult/ls/rs broadcast along the last axis.  Implemented with Python ints to stay exact."""
    acc = np.asarray(acc, dtype=np.int64)
    flat = acc.reshape(-1, acc.shape[-1])
    out = np.empty_like(flat)
    for c in range(flat.shape[1]):
        m, l, r = int(mult[c]), int(ls[c]), int(rs[c])
        col = flat[:, c]
        out[:, c] = [min(max(wrap32(mbqm(int(v), m, l, r) + zo), amin), amax) for v in col]
    return out.reshape(acc.shape)


def matmul_int8(a, w_nk, bias, sx, zx, sw, zw, so, zo, act):
    """sum_k (x - zx)(w - zw) + bias, wrapped to int32, requantised.  w_nk is [N, K]."""
    a64 = a.astype(np.int64)
    w64 = w_nk.astype(np.int64)
    n = w64.shape[0]
    zw = np.broadcast_to(np.atleast_1d(np.asarray(zw, dtype=np.int64)), (n,)) if np.size(zw) == 1 else np.asarray(zw, np.int64)
    acc = (a64 - zx) @ (w64 - zw[:, None]).T
    if bias is not None:
        acc = acc + bias.astype(np.int64)[None, :]
    acc = wrap32(acc)
    sw = np.atleast_1d(sw)
    mult, ls, rs = requant_params(sx, sw, so)
    if len(sw) == 1:
        mult, ls, rs = (np.repeat(v, n) for v in (mult, ls, rs))
    lo, hi = act_range(act == 1, act == 3, zo, so)
    return requant_vec(acc, mult, ls, rs, zo, lo, hi).astype(np.int8)


def conv_int8(x, w, bias, shape, sx, zx, sw, zw, so, zo, act, depthwise=False):
    """Direct NHWC convolution of (x - zx) with (w - zw); taps outside the image contribute nothing, except for a
    1x1 kernel with stride/pad where the reference feeds literal zeros (contribution (0 - zx)(w - zw))."""
    b, ih, iw, ic = x.shape
    oh, ow, oc = shape.out_h, shape.out_w, shape.out_c
    kh, kw = shape.kernel_h, shape.kernel_w
    zw = np.asarray(zw, np.int64)
    zwv = np.repeat(zw, oc) if zw.size == 1 else zw
    is_1x1 = (kh == 1 and kw == 1) and not depthwise
    acc = np.zeros((b, oh, ow, oc), np.int64)
    xs = x.astype(np.int64) - zx
    for r in range(kh):
        for c in range(kw):
            for y in range(oh):
                iy = y * shape.stride_h - shape.pad_u + r * shape.dilation_h
                for xx in range(ow):
                    ix = xx * shape.stride_w - shape.pad_l + c * shape.dilation_w
                    inside = 0 <= iy < ih and 0 <= ix < iw
                    if inside:
                        px = xs[:, iy, ix, :]
                    elif is_1x1:
                        px = np.full((b, ic), -zx, np.int64)
                    else:
                        continue
                    if depthwise:
                        wt = w[:, r, c].astype(np.int64) - zwv  # [C]
                        acc[:, y, xx, :] += px * wt[None, :]
                    else:
                        wt = w[:, r, c, :].astype(np.int64) - zwv[:, None]  # [OC, IC]
                        acc[:, y, xx, :] += px @ wt.T
    if bias is not None:
        acc += bias.astype(np.int64)
    acc = wrap32(acc)
    sw = np.atleast_1d(sw)
    mult, ls, rs = requant_params(sx, sw, so)
    if len(sw) == 1:
        mult, ls, rs = (np.repeat(v, oc) for v in (mult, ls, rs))
    lo, hi = act_range(act == 1, act == 3, zo, so)
    return requant_vec(acc, mult, ls, rs, zo, lo, hi).astype(np.int8)


def dynquant_params(x, symmetric=False):
    x = np.asarray(x, np.float32)
    finite_or_inf = x[~np.isnan(x)]
    mn = np.float32(finite_or_inf.min()) if finite_or_inf.size else np.float32(np.finfo(np.float32).max)
    mx = np.float32(finite_or_inf.max()) if finite_or_inf.size else np.float32(-np.finfo(np.float32).max)
    mn = min(mn, np.float32(np.finfo(np.float32).max))
    mx = max(mx, np.float32(-np.finfo(np.float32).max))
    if not symmetric:
        rng = np.float32(mx - mn)
        if rng <= 0:
            rng = np.float32(0.01)
        scale = np.float64(np.float32(rng / np.float32(255.0)))
        zp = int(round_half_away(np.float64(-128.0) - np.float64(mn) / scale))
    else:
        big = max(abs(mx), abs(mn))
        scale = np.float64(np.float32(np.float32(np.float32(2.0) * big) / np.float32(254.0)))
        zp = 0
    return float(scale), zp


def quantize_fp32_int8(x, scale, zp):
    x = np.asarray(x, np.float32)
    inv = np.float32(1.0) / np.float32(scale)
    with np.errstate(all="ignore"):
        t = (x * inv).astype(np.float32) + np.float32(zp)
        r = round_half_away(t.astype(np.float64))
    bad = ~(np.abs(r) < 2147483648.0)  # NaN or beyond int32 -> INT_MIN on x86
    r = np.where(bad, -2147483648.0, r)
    q = np.clip(r, -128, 127)
    q = np.where(x == np.inf, 127, q)
    q = np.where(x == -np.inf, -128, q)
    return q.astype(np.int8)


def dynamic_matmul(a, w_nk, bias, sx, zx, sw, zw0, act):
    a64, w64 = a.astype(np.int64), w_nk.astype(np.int64)
    value = wrap32((a64 - zx) @ (w64 - zw0).T)
    sw = np.atleast_1d(sw)
    ms = (np.float32(sx) * sw.astype(np.float32)).astype(np.float32)
    if ms.size == 1:
        ms = np.repeat(ms, w64.shape[0])
    d = (ms[None, :] * value.astype(np.float32)).astype(np.float32)
    if bias is not None:
        d = (d + bias.astype(np.float32)[None, :]).astype(np.float32)
    if act == 1:
        d = np.where(0 > d, np.float32(0), d)
    elif act == 3:
        d = np.where(0 > d, np.float32(0), d)
        d = np.where(6 < d, np.float32(6), d)
    return d.astype(np.float32)
