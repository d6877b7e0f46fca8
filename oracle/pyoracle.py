"""TEST INFRASTRUCTURE ONLY: ctypes bindings for the two CPU checkers.

* ``Oracle``    -- ``oracle/liboracle.so``, the from-scratch restatement (``nnacl_restate.c``).
* ``Reference`` -- ``oracle/_ref/libnnacl_ref.so``, the real nnacl kernels compiled from the reference tree plus
  the wrapper call sequences of ``ref_driver.c``.  May be absent (then ``Reference.available()`` is False).

Only tests, the smoke entry and the benchmark's ``cpu_baseline`` leg may import this module.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libnnacl_ref.so")

ACT_NONE, ACT_RELU, ACT_RELU6 = 0, 1, 3


class ConvShape(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "batch", "in_h", "in_w", "in_c", "out_h", "out_w", "out_c", "kernel_h", "kernel_w", "stride_h", "stride_w",
        "dilation_h", "dilation_w", "pad_u", "pad_l")]


def conv_shape(batch, in_h, in_w, in_c, out_c, kernel, stride=(1, 1), dilation=(1, 1), pad=(0, 0, 0, 0)):
    """pad = (up, down, left, right); output size follows the usual floor formula."""
    kh, kw = kernel
    sh, sw = stride
    dh, dw = dilation
    pu, pd, pl, pr = pad
    oh = (in_h + pu + pd - ((kh - 1) * dh + 1)) // sh + 1
    ow = (in_w + pl + pr - ((kw - 1) * dw + 1)) // sw + 1
    return ConvShape(batch, in_h, in_w, in_c, oh, ow, out_c, kh, kw, sh, sw, dh, dw, pu, pl)


def _p(a, t):
    return None if a is None else a.ctypes.data_as(C.POINTER(t))


def _i8(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int8)


def _i32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _f64(a):
    return np.ascontiguousarray(np.atleast_1d(a), dtype=np.float64)


class _Base:
    prefix = ""
    extra = False  # driver entry points take (threads, run_seconds*)

    def __init__(self, path):
        self.lib = C.CDLL(path)
        self.threads = 1
        self.last_seconds = 0.0

    def _tail(self):
        if not self.extra:
            return []
        self._secs = C.c_double(0.0)
        return [C.c_int(self.threads), C.byref(self._secs)]

    def _done(self, rc, what):
        if self.extra:
            self.last_seconds = self._secs.value
        if rc != 0:
            raise RuntimeError("%s%s failed: %d" % (self.prefix, what, rc))

    def matmul_int8(self, a, w, bias, sx, zx, sw, zw, so, zo, act=ACT_NONE, b_transpose=True):
        a, w, bias = _i8(a), _i8(w), _i32(bias)
        m, k = a.shape
        n = w.shape[0] if b_transpose else w.shape[1]
        sw, zw = _f64(sw), _i32(np.atleast_1d(zw))
        out = np.empty((m, n), np.int8)
        f = getattr(self.lib, self.prefix + "matmul_int8")
        f.restype = C.c_int
        rc = f(_p(a, C.c_int8), _p(w, C.c_int8), _p(bias, C.c_int32), _p(out, C.c_int8), C.c_int(m), C.c_int(n),
               C.c_int(k), C.c_int(1 if b_transpose else 0), C.c_double(sx), C.c_int(zx), _p(sw, C.c_double),
               _p(zw, C.c_int32), C.c_int(len(sw)), C.c_double(so), C.c_int(zo), C.c_int(act), *self._tail())
        self._done(rc, "matmul_int8")
        return out

    def _conv(self, name, x, w, bias, shape, sx, zx, sw, zw, so, zo, act):
        x, w, bias = _i8(x), _i8(w), _i32(bias)
        sw, zw = _f64(sw), _i32(np.atleast_1d(zw))
        out = np.empty((shape.batch, shape.out_h, shape.out_w, shape.out_c), np.int8)
        f = getattr(self.lib, self.prefix + name)
        f.restype = C.c_int
        rc = f(_p(x, C.c_int8), _p(w, C.c_int8), _p(bias, C.c_int32), _p(out, C.c_int8), C.byref(shape),
               C.c_double(sx), C.c_int(zx), _p(sw, C.c_double), _p(zw, C.c_int32), C.c_int(len(sw)), C.c_double(so),
               C.c_int(zo), C.c_int(act), *self._tail())
        self._done(rc, name)
        return out

    def conv_int8(self, x, w, bias, shape, sx, zx, sw, zw, so, zo, act=ACT_NONE):
        return self._conv("conv_int8", x, w, bias, shape, sx, zx, sw, zw, so, zo, act)

    def conv_int8_as_arm64_sdot(self, x, w, bias, shape, sx, zx, sw, zw, so, zo, act=ACT_NONE):
        """ConvInt8 whatever the kernel size: the compiled reference refuses dense 3x3 stride-1 convolutions through
        conv_int8 (x86 selects a Winograd kernel for them), this entry runs ConvInt8 on them as ARM64 cores with dot
        product do.  The restatement computes the exact convolution either way."""
        name = "conv_int8_as_arm64_sdot" if self.prefix == "ref_" else "conv_int8"
        return self._conv(name, x, w, bias, shape, sx, zx, sw, zw, so, zo, act)

    def conv_dw_int8(self, x, w, bias, shape, sx, zx, sw, zw, so, zo, act=ACT_NONE):
        return self._conv("conv_dw_int8", x, w, bias, shape, sx, zx, sw, zw, so, zo, act)

    def dynamic_quant(self, x, symmetric=False):
        x = _f32(x)
        q = np.empty(x.shape, np.int8)
        scale, zp = C.c_double(0), C.c_int32(0)
        f = getattr(self.lib, self.prefix + "dynamic_quant")
        f.restype = C.c_int
        n = C.c_int(x.size) if self.extra else C.c_int64(x.size)
        rc = f(_p(x, C.c_float), n, C.c_int(1 if symmetric else 0), _p(q, C.c_int8), C.byref(scale), C.byref(zp),
               *self._tail())
        self._done(rc, "dynamic_quant")
        return q, scale.value, zp.value

    def dynamic_quant_segments(self, x, symmetric=False):
        """x: [segments, unit] fp32 (the layout after the preferred axes lead) -> (q, scales[segments], zps)."""
        x = _f32(x)
        segments, unit = x.shape
        q = np.empty(x.shape, np.int8)
        scales, zps = np.empty(segments, np.float64), np.empty(segments, np.int32)
        f = getattr(self.lib, self.prefix + "dynamic_quant_segments")
        f.restype = C.c_int
        it = C.c_int if self.extra else C.c_int64
        rc = f(_p(x, C.c_float), it(segments), it(unit), C.c_int(1 if symmetric else 0), _p(q, C.c_int8),
               _p(scales, C.c_double), _p(zps, C.c_int32), *self._tail())
        self._done(rc, "dynamic_quant_segments")
        return q, scales, zps

    def dynamic_matmul_rows(self, a, w, bias, sx_rows, zx, sw, zw, act=ACT_NONE, b_transpose=True):
        """Per-row input scales (float32 [rows]), one input zero point."""
        a, w, bias, sx_rows = _i8(a), _i8(w), _f32(bias), _f32(sx_rows)
        m, k = a.shape
        n = w.shape[0] if b_transpose else w.shape[1]
        sw, zw = _f64(sw), _i32(np.atleast_1d(zw))
        out = np.empty((m, n), np.float32)
        f = getattr(self.lib, self.prefix + "dynamic_matmul_rows")
        f.restype = C.c_int
        rc = f(_p(a, C.c_int8), _p(w, C.c_int8), _p(bias, C.c_float), _p(out, C.c_float), C.c_int(m), C.c_int(n),
               C.c_int(k), C.c_int(1 if b_transpose else 0), _p(sx_rows, C.c_float), C.c_int(zx), _p(sw, C.c_double),
               _p(zw, C.c_int32), C.c_int(len(sw)), C.c_int(act), *self._tail())
        self._done(rc, "dynamic_matmul_rows")
        return out

    def dynamic_matmul(self, a, w, bias, sx, zx, sw, zw, act=ACT_NONE, b_transpose=True):
        a, w, bias = _i8(a), _i8(w), _f32(bias)
        m, k = a.shape
        n = w.shape[0] if b_transpose else w.shape[1]
        sw, zw = _f64(sw), _i32(np.atleast_1d(zw))
        out = np.empty((m, n), np.float32)
        f = getattr(self.lib, self.prefix + "dynamic_matmul")
        f.restype = C.c_int
        rc = f(_p(a, C.c_int8), _p(w, C.c_int8), _p(bias, C.c_float), _p(out, C.c_float), C.c_int(m), C.c_int(n),
               C.c_int(k), C.c_int(1 if b_transpose else 0), C.c_double(sx), C.c_int(zx), _p(sw, C.c_double),
               _p(zw, C.c_int32), C.c_int(len(sw)), C.c_int(act), *self._tail())
        self._done(rc, "dynamic_matmul")
        return out


class Oracle(_Base):
    prefix = "orc_"

    def __init__(self, path=ORACLE_SO):
        super().__init__(path)
        L = self.lib
        L.orc_srdhm.restype = C.c_int32
        L.orc_srdhm.argtypes = [C.c_int32, C.c_int32]
        L.orc_rdiv_pot.restype = C.c_int32
        L.orc_rdiv_pot.argtypes = [C.c_int32, C.c_int32]
        L.orc_mul_by_quant_mult.restype = C.c_int32
        L.orc_mul_by_quant_mult.argtypes = [C.c_int32] * 4
        L.orc_set_threads.argtypes = [C.c_int]

    def set_threads(self, n):
        self.threads = n
        self.lib.orc_set_threads(n)

    def srdhm(self, a, b):
        return self.lib.orc_srdhm(a, b)

    def rdiv_pot(self, x, e):
        return self.lib.orc_rdiv_pot(x, e)

    def mul_by_quant_mult(self, v, mult, ls, rs):
        return self.lib.orc_mul_by_quant_mult(v, mult, ls, rs)

    def quantize_multiplier(self, m):
        mult, shift = C.c_int32(0), C.c_int32(0)
        self.lib.orc_quantize_multiplier(C.c_double(m), C.byref(mult), C.byref(shift))
        return mult.value, shift.value

    def round_param(self, m):
        mult, ls, rs = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self.lib.orc_round_param(C.c_double(m), C.byref(mult), C.byref(ls), C.byref(rs))
        return mult.value, ls.value, rs.value

    def round_param_single(self, m):
        mult, ls, rs = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self.lib.orc_round_param_single(C.c_double(m), C.byref(mult), C.byref(ls), C.byref(rs))
        return mult.value, ls.value, rs.value

    def act_range(self, relu, relu6, zp, scale):
        mn, mx = C.c_int32(0), C.c_int32(0)
        self.lib.orc_act_range(C.c_int(relu), C.c_int(relu6), C.c_int32(zp), C.c_float(scale), C.byref(mn),
                               C.byref(mx))
        return mn.value, mx.value

    def requant_params(self, sx, sw, so):
        sw = _f64(sw)
        n = len(sw)
        mult, ls, rs = (np.empty(n, np.int32) for _ in range(3))
        self.lib.orc_requant_params(C.c_double(sx), _p(sw, C.c_double), C.c_int(n), C.c_double(so),
                                    _p(mult, C.c_int32), _p(ls, C.c_int32), _p(rs, C.c_int32))
        return mult, ls, rs

    def minmax(self, x):
        x = _f32(x)
        mn, mx = C.c_float(np.finfo(np.float32).max), C.c_float(-np.finfo(np.float32).max)
        self.lib.orc_minmax_fp32(_p(x, C.c_float), C.c_int64(x.size), C.byref(mn), C.byref(mx))
        return mn.value, mx.value

    def dynquant_params(self, mn, mx, symmetric=False):
        scale, zp = C.c_double(0), C.c_int32(0)
        self.lib.orc_dynquant_params(C.c_float(mn), C.c_float(mx), C.c_int(1 if symmetric else 0), C.byref(scale),
                                     C.byref(zp))
        return scale.value, zp.value

    def quantize_fp32_int8(self, x, scale, zp):
        x = _f32(x)
        q = np.empty(x.shape, np.int8)
        self.lib.orc_quantize_fp32_int8(_p(x, C.c_float), _p(q, C.c_int8), C.c_float(scale), C.c_int32(zp),
                                        C.c_int64(x.size))
        return q


class Reference(_Base):
    """The compiled nnacl kernels + wrapper call sequences (x86 non-ARM branches)."""
    prefix = "ref_"
    extra = True

    def __init__(self, path=REF_SO):
        super().__init__(path)
        L = self.lib
        L.SaturatingRoundingDoublingHighMul.restype = C.c_int
        L.SaturatingRoundingDoublingHighMul.argtypes = [C.c_int, C.c_int]
        L.RoundingDivideByPOT.restype = C.c_int
        L.RoundingDivideByPOT.argtypes = [C.c_int, C.c_int]
        L.MultiplyByQuantizedMultiplier.restype = C.c_int
        L.MultiplyByQuantizedMultiplier.argtypes = [C.c_int32] * 4

    @staticmethod
    def available():
        return os.path.exists(REF_SO)

    def srdhm(self, a, b):
        return self.lib.SaturatingRoundingDoublingHighMul(a, b)

    def rdiv_pot(self, x, e):
        return self.lib.RoundingDivideByPOT(x, e)

    def mul_by_quant_mult(self, v, mult, ls, rs):
        return self.lib.MultiplyByQuantizedMultiplier(v, mult, ls, rs)

    def quantize_multiplier(self, m):
        mult, shift = C.c_int32(0), C.c_int(0)
        self.lib.QuantizeMultiplier(C.c_double(m), C.byref(mult), C.byref(shift))
        return mult.value, shift.value

    def round_param(self, m):
        mult, ls, rs = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self.lib.QuantizeRoundParameterWithDoublePrecision(C.c_double(m), C.byref(mult), C.byref(ls), C.byref(rs))
        return mult.value, ls.value, rs.value

    def round_param_single(self, m):
        mult, ls, rs = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        self.lib.QuantizeRoundParameterWithSinglePrecision(C.c_double(m), C.byref(mult), C.byref(ls), C.byref(rs))
        return mult.value, ls.value, rs.value

    def act_range(self, relu, relu6, zp, scale):
        mn, mx = C.c_int32(0), C.c_int32(0)
        self.lib.CalculateActivationRangeQuantized(C.c_bool(relu), C.c_bool(relu6), C.c_int32(zp), C.c_float(scale),
                                                   C.byref(mn), C.byref(mx))
        return mn.value, mx.value

    # ---- shape inference: the real nnacl functions; status is "ok", "invalid" (unknown dimension) or "error" ----
    def _infer_status(self, ret):
        return "ok" if ret == 0 else "invalid" if ret == self.lib.ref_nnacl_infer_invalid() else "error"

    @staticmethod
    def _ishape(shape):
        shape = [] if shape is None else [int(d) for d in shape]
        return (C.c_int * max(len(shape), 1))(*shape), len(shape)

    def infer_matmul(self, a_shape, b_shape, bias_shape=None, transpose_a=False, transpose_b=False):
        a, an = self._ishape(a_shape)
        b, bn = self._ishape(b_shape)
        bias, biasn = self._ishape(bias_shape)
        out, on = (C.c_int * 8)(), C.c_int(0)
        ret = self.lib.ref_infer_matmul(a, an, b, bn, bias, biasn, int(transpose_a), int(transpose_b), out,
                                        C.byref(on))
        return self._infer_status(ret), [out[i] for i in range(min(on.value, 8))]

    def infer_fullconnection(self, a_shape, w_shape, bias_shape=None, has_bias=False, use_axis=False, axis=0):
        a, an = self._ishape(a_shape)
        w, wn = self._ishape(w_shape)
        bias, biasn = self._ishape(bias_shape)
        out, on = (C.c_int * 8)(), C.c_int(0)
        ret = self.lib.ref_infer_fullconnection(a, an, w, wn, bias, biasn, int(has_bias), int(use_axis), int(axis),
                                                out, C.byref(on))
        return self._infer_status(ret), [out[i] for i in range(min(on.value, 8))]

    def infer_conv2d(self, in_shape, w_shape, kernel, stride, dilation, pad_mode, pads, group):
        x, xn = self._ishape(in_shape)
        w, wn = self._ishape(w_shape)
        cp = (C.c_int * 12)(kernel[0], kernel[1], stride[0], stride[1], dilation[0], dilation[1], pad_mode,
                            pads[0], pads[1], pads[2], pads[3], group)
        out, on = (C.c_int * 8)(), C.c_int(0)
        ret = self.lib.ref_infer_conv2d(x, xn, w, wn, cp, out, C.byref(on))
        return (self._infer_status(ret), [out[i] for i in range(min(on.value, 8))], tuple(cp[7:11]),
                (cp[0], cp[1]), cp[11])

    def minmax(self, x):
        x = _f32(x)
        mn, mx = C.c_float(np.finfo(np.float32).max), C.c_float(-np.finfo(np.float32).max)
        self.lib.CalculateMinMaxFp32(_p(x, C.c_float), C.c_int(x.size), C.byref(mn), C.byref(mx))
        return mn.value, mx.value

    def quantize_fp32_int8(self, x, scale, zp):
        x = _f32(x)
        q = np.empty(x.shape, np.int8)
        self.lib.DoQuantizeFp32ToInt8(_p(x, C.c_float), _p(q, C.c_int8), C.c_float(scale), C.c_int32(zp),
                                      C.c_int(x.size), C.c_int32(-128), C.c_int32(127))
        return q


_oracle = None
_reference = None


def pack_weight_4x16(w_nk):
    """The offline weight layout of MatMulDynamicSdotInt8Kernel for a weight given as [N][K]: blocks
    [N / 16][K / 4][16 channels][4 K-bytes], N padded to 16 and K to 4 with zeros.  Restates
    RowMajor2Row4x16MajorInt8 (on the [N, K] weight of transpose_b) and RowMajor2Col4x16MajorInt8 (on its [K, N]
    transpose), nnacl/int8/matmul_int8.c:143-156 and :770-784, which produce the same bytes."""
    w_nk = np.ascontiguousarray(w_nk, dtype=np.int8)
    n, k = w_nk.shape
    n16, k4 = -(-n // 16) * 16, -(-k // 4) * 4
    padded = np.zeros((n16, k4), np.int8)
    padded[:n, :k] = w_nk
    return np.ascontiguousarray(padded.reshape(n16 // 16, 16, k4 // 4, 4).transpose(0, 2, 1, 3)).reshape(-1)


def broadcast_offsets(a_shape, b_shape):
    """(a_offsets, b_offsets) per output matrix of a batched MatMul: restates
    MatmulFp32BaseCPUKernel::InitBroadcastParams (mindspore/lite/src/litert/kernel/cpu/fp32/matmul_fp32_base.cc:
    576-646) in the terms of NumPy broadcasting over the batch axes, with the reference's extension that a batch
    extent may divide the other operand's (index scaled proportionally)."""
    rank = max(len(a_shape), len(b_shape), 4)
    a = [1] * (rank - len(a_shape)) + list(a_shape)
    b = [1] * (rank - len(b_shape)) + list(b_shape)
    nb = rank - 2
    mx = [max(a[j], b[j]) for j in range(nb)]
    for j in range(nb):
        mn = max(min(a[j], b[j]), 1)
        if mx[j] != mn and mx[j] % mn != 0:
            raise ValueError("batch extents %d and %d cannot be broadcast" % (a[j], b[j]))
    a_off, b_off = [], []
    for idx in np.ndindex(*mx) if nb else [()]:
        ao = bo = 0
        for j in range(nb):
            ao = ao * a[j] + idx[j] * a[j] // mx[j]
            bo = bo * b[j] + idx[j] * b[j] // mx[j]
        a_off.append(ao)
        b_off.append(bo)
    return a_off, b_off


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            raise RuntimeError("oracle/liboracle.so is not built: run `make -C oracle` (or __graft_entry__.build())")
        _oracle = Oracle()
    return _oracle


def reference():
    global _reference
    if _reference is None:
        _reference = Reference()
    return _reference
