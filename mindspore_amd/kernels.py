"""Host-side mirror of the Lite int8 kernel wrappers over the C ABI.

Each class plays the role of one reference CPU kernel class (same inputs, same quant-parameter meaning, same error
behaviour: construction = Prepare(), ``run`` = Run()):

  MatmulInt8Kernel / FullconnectionInt8Kernel  <-  MatmulInt8CPUKernel / FullconnectionInt8CPUKernel
  ConvolutionInt8Kernel                        <-  Convolution1x1Int8 / ConvolutionInt8 / ConvolutionDepthwiseInt8
  DynamicQuantKernel                           <-  DynamicQuantCPUKernel
  MatmulDynamicInt8Kernel                      <-  MatmulDynamicInt8CPUKernel

``run`` accepts either NumPy arrays (host tensors: copied to the GPU, computed, copied back) or torch CUDA tensors
(device tensors: computed in place on torch's current stream, no copies).  torch is only used as a device-memory
and stream provider.
"""
import ctypes as C
from collections import namedtuple

import numpy as np

from . import lib as _lib

QuantParam = namedtuple("QuantParam", ["scale", "zero_point"])
ACT_NONE, ACT_RELU, ACT_RELU6 = _lib.ACT_NONE, _lib.ACT_RELU, _lib.ACT_RELU6


def _is_torch(x):
    return type(x).__module__.startswith("torch")


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _quant_arrays(params):
    params = list(params)
    if not params:
        raise ValueError("at least one weight quant param is required")
    scales = (C.c_double * len(params))(*[float(p.scale) for p in params])
    zps = (C.c_int32 * len(params))(*[int(p.zero_point) for p in params])
    return len(params), scales, zps


def _host_i8(a):
    a = np.ascontiguousarray(a)
    if a.dtype != np.int8:
        raise TypeError("expected an int8 tensor, got %s" % a.dtype)
    return a


class _Handle:
    _destroy = None

    def __init__(self):
        self._h = C.c_void_p(None)

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            getattr(_lib.load(), self._destroy)(self._h)
            self._h = C.c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class MatmulInt8Kernel(_Handle):
    """Full-quant int8 MatMul: C = requant(A x W^T).  weight is [N, K] when transpose_b else [K, N]; bias int32 [N].
    decode_pack=False skips the second packed form of the weights (the one runs with 2..64 rows use, 2..128 against at most 4096 channels with K >= 1024); such rows then
    run on the GEMM tiles."""
    _destroy = "mi_matmul_destroy"

    def __init__(self, weight, bias, in_quant, weight_quant, out_quant, transpose_b=True, act=ACT_NONE, device=0,
                 decode_pack=True):
        super().__init__()
        L = _lib.init(device)
        weight = _host_i8(weight)
        if weight.ndim < 2:
            raise ValueError("weight must have at least two dimensions")
        # a constant weight of rank > 2 is a batch of matrices (matmul_base_int8.cc:366-368)
        self.w_shape = tuple(weight.shape)
        self.b_batch = int(np.prod(weight.shape[:-2])) if weight.ndim > 2 else 1
        self.n, self.k = (weight.shape[-2:] if transpose_b else weight.shape[-2:][::-1])
        self.transpose_b = bool(transpose_b)
        if bias is not None:
            bias = np.ascontiguousarray(bias)
            if bias.dtype != np.int32:
                raise TypeError("full-quant MatMul needs an int32 bias")  # matmul_base_int8.cc:420-424
            if bias.size != self.n:
                raise ValueError("bias has %d entries, expected %d" % (bias.size, self.n))
        nq, scales, zps = _quant_arrays(weight_quant)
        d = _lib.MatmulDesc(self.k, self.n, 1 if transpose_b else 0, act, float(in_quant.scale),
                            int(in_quant.zero_point), float(out_quant.scale), int(out_quant.zero_point), nq, scales,
                            zps, 0 if decode_pack else _lib.MATMUL_NO_DECODE_PACK, self.b_batch)
        _lib.check(L.mi_matmul_create(C.byref(d), weight.ctypes.data, None if bias is None else bias.ctypes.data,
                                      C.byref(self._h)), "mi_matmul_create")

    def run(self, a, out=None):
        """a: int8 [..., K] as a numpy array (host path) or a contiguous CUDA tensor (device path, current stream).
        `out` (device path only) is a preallocated contiguous CUDA int8 tensor [..., N] to write into."""
        L = _lib.load()
        if _is_torch(a):
            import torch
            if a.dtype != torch.int8 or not a.is_cuda or not a.is_contiguous() or a.shape[-1] != self.k:
                raise ValueError("expected a contiguous CUDA int8 tensor [..., %d]" % self.k)
            rows = a.numel() // self.k
            if out is None:
                out = torch.empty(a.shape[:-1] + (self.n,), dtype=torch.int8, device=a.device)
            elif (out.dtype != torch.int8 or not out.is_cuda or not out.is_contiguous()
                  or out.numel() != rows * self.n):
                raise ValueError("out must be a contiguous CUDA int8 tensor with %d elements" % (rows * self.n))
            _lib.check(L.mi_matmul_run(self._h, a.data_ptr(), rows, out.data_ptr(), _stream()), "mi_matmul_run")
            return out
        a = _host_i8(a)
        if a.shape[-1] != self.k:
            raise ValueError("expected [..., %d], got %s" % (self.k, a.shape))
        rows = a.size // self.k
        out = np.empty(a.shape[:-1] + (self.n,), np.int8)
        _lib.check(L.mi_matmul_run_host(self._h, a.ctypes.data, rows, out.ctypes.data), "mi_matmul_run_host")
        return out

    def run_batched(self, a):
        """Batched MatMul against a weight of rank > 2 (or a rank-2 weight broadcast over a batched `a`): a is a
        contiguous CUDA int8 tensor [..., rows, K]; the batch extents of `a` and of the weight are broadcast as the
        reference does (MatmulFp32BaseCPUKernel::InitBroadcastParams).  Returns [batch..., rows, N]."""
        import torch
        L = _lib.load()
        if a.dtype != torch.int8 or not a.is_cuda or not a.is_contiguous() or a.ndim < 2 or a.shape[-1] != self.k:
            raise ValueError("expected a contiguous CUDA int8 tensor [..., rows, %d]" % self.k)
        rows = a.shape[-2]
        a_shape, an = _shape_arg(a.shape)
        w_shape, wn = _shape_arg(self.w_shape)
        cap = 1 << 16
        batch = C.c_int32(0)
        a_off, b_off = (C.c_int32 * cap)(), (C.c_int32 * cap)()
        _lib.check(L.mi_matmul_broadcast_offsets(a_shape, an, w_shape, wn, cap, C.byref(batch), a_off, b_off),
                   "mi_matmul_broadcast_offsets")
        rank = max(a.ndim, len(self.w_shape))
        ash = (1,) * (rank - a.ndim) + tuple(a.shape)
        wsh = (1,) * (rank - len(self.w_shape)) + self.w_shape
        out_shape = tuple(max(x, y) for x, y in zip(ash[:-2], wsh[:-2])) + (rows, self.n)
        out = torch.empty(out_shape, dtype=torch.int8, device=a.device)
        _lib.check(L.mi_matmul_run_batched(self._h, a.data_ptr(), rows, batch.value, a_off, b_off, out.data_ptr(),
                                           _stream()), "mi_matmul_run_batched")
        return out

    def reserve(self, max_rows):
        """ReSize(): sizes the workspaces so that runs of up to max_rows rows allocate nothing."""
        _lib.check(_lib.load().mi_matmul_reserve(self._h, int(max_rows)), "mi_matmul_reserve")

    def params(self):
        L = _lib.load()
        arrs = [np.empty(self.n, np.int32) for _ in range(4)]
        lo, hi = C.c_int32(0), C.c_int32(0)
        _lib.check(L.mi_matmul_get_params(self._h, *[x.ctypes.data for x in arrs], C.byref(lo), C.byref(hi)),
                   "mi_matmul_get_params")
        return dict(multiplier=arrs[0], left_shift=arrs[1], right_shift=arrs[2], folded_bias=arrs[3],
                    act_min=lo.value, act_max=hi.value)


class FullconnectionInt8Kernel(MatmulInt8Kernel):
    """FullConnection always uses a [N, K] weight (fullconnection_int8.cc:33-34)."""

    def __init__(self, weight, bias, in_quant, weight_quant, out_quant, act=ACT_NONE, device=0):
        super().__init__(weight, bias, in_quant, weight_quant, out_quant, True, act, device)


def matmul_run_group(kernels, a, outs=None):
    """Runs several MatmulInt8Kernel objects that share the input `a` (a contiguous CUDA int8 tensor [..., K]) as
    mi_matmul_run_group does: decode-sized inputs go out as one launch.  Returns the list of outputs."""
    import torch
    L = _lib.load()
    k = kernels[0].k
    if a.dtype != torch.int8 or not a.is_cuda or not a.is_contiguous() or a.shape[-1] != k:
        raise ValueError("expected a contiguous CUDA int8 tensor [..., %d]" % k)
    rows = a.numel() // k
    if outs is None:
        outs = [torch.empty(a.shape[:-1] + (kn.n,), dtype=torch.int8, device=a.device) for kn in kernels]
    hs = (C.c_void_p * len(kernels))(*[kn._h.value for kn in kernels])
    cs = (C.c_void_p * len(kernels))(*[o.data_ptr() for o in outs])
    _lib.check(L.mi_matmul_run_group(hs, len(kernels), a.data_ptr(), rows, cs, _stream()), "mi_matmul_run_group")
    return outs


def dynmm_run_group(kernels, a, in_quant=None, params_dev=None, row_params=None, outs=None):
    """Runs several MatmulDynamicInt8Kernel objects that share the input `a` (a contiguous CUDA int8 tensor [..., K])
    as mi_dynmm_run_group does: decode-sized inputs go out as one launch.  The input's quantisation comes as one
    QuantParam (in_quant), as the address of the block a DynamicQuantKernel.run left on the device (params_dev) or as
    the tensor DynamicQuantKernel.run_rows returned (row_params).  Returns the list of fp32 outputs."""
    import torch
    L = _lib.load()
    k = kernels[0].k
    if a.dtype != torch.int8 or not a.is_cuda or not a.is_contiguous() or a.shape[-1] != k:
        raise ValueError("expected a contiguous CUDA int8 tensor [..., %d]" % k)
    rows = a.numel() // k
    if outs is None:
        outs = [torch.empty(a.shape[:-1] + (kn.n,), dtype=torch.float32, device=a.device) for kn in kernels]
    hs = (C.c_void_p * len(kernels))(*[kn._h.value for kn in kernels])
    cs = (C.c_void_p * len(kernels))(*[o.data_ptr() for o in outs])
    scale, zp, dev, per_row = 0.0, 0, None, 0
    if row_params is not None:
        dev, per_row = row_params.data_ptr(), 1
    elif params_dev is not None:
        dev = params_dev
    else:
        scale, zp = float(in_quant.scale), int(in_quant.zero_point)
    _lib.check(L.mi_dynmm_run_group(hs, len(kernels), a.data_ptr(), rows, scale, zp, dev, per_row, cs, _stream()),
               "mi_dynmm_run_group")
    return outs


class ConvolutionInt8Kernel(_Handle):
    """Conv2DFusion int8, NHWC.  weight [OC, KH, KW, IC] (group 1) or [C, KH, KW] (depthwise, group == C).
    pad = (up, down, left, right).  Raises MiError with code MI_NOT_SUPPORT for the cases a provider must decline.
    exact_3x3: take dense 3x3 stride-1 convolutions too, computing the exact convolution as the reference does on
    ARM64 cores with dot-product instructions (other builds of the reference run an integer Winograd there)."""
    _destroy = "mi_conv_destroy"

    def __init__(self, weight, bias, in_quant, weight_quant, out_quant, stride=(1, 1), dilation=(1, 1),
                 pad=(0, 0, 0, 0), group=1, act=ACT_NONE, device=0, exact_3x3=False):
        super().__init__()
        L = _lib.init(device)
        weight = _host_i8(weight)
        if group == 1:
            if weight.ndim != 4:
                raise ValueError("weight must be [OC, KH, KW, IC]")
            oc, kh, kw, ic = weight.shape
        else:
            if weight.ndim == 4 and weight.shape[3] == 1:
                weight = weight.reshape(weight.shape[:3])
            if weight.ndim != 3:
                raise ValueError("depthwise weight must be [C, KH, KW]")
            oc, kh, kw = weight.shape
            ic = oc
        if bias is not None:
            bias = np.ascontiguousarray(bias)
            if bias.dtype != np.int32 or bias.size != oc:
                raise ValueError("bias must be int32 [%d]" % oc)
        self.ic, self.oc = ic, oc
        nq, scales, zps = _quant_arrays(weight_quant)
        d = _lib.ConvDesc(ic, oc, kh, kw, stride[0], stride[1], dilation[0], dilation[1], pad[0], pad[1], pad[2],
                          pad[3], group, act, float(in_quant.scale), int(in_quant.zero_point),
                          float(out_quant.scale), int(out_quant.zero_point), nq, scales, zps,
                          _lib.CONV_3X3_EXACT if exact_3x3 else 0)
        _lib.check(L.mi_conv_create(C.byref(d), weight.ctypes.data, None if bias is None else bias.ctypes.data,
                                    C.byref(self._h)), "mi_conv_create")

    def out_shape(self, in_h, in_w):
        oh, ow = C.c_int32(0), C.c_int32(0)
        _lib.check(_lib.load().mi_conv_out_shape(self._h, in_h, in_w, C.byref(oh), C.byref(ow)), "mi_conv_out_shape")
        return oh.value, ow.value

    def run(self, x, out=None):
        """x: int8 NHWC as a numpy array (host path) or a contiguous CUDA tensor (device path, current stream);
        `out` (device path only) is a preallocated contiguous CUDA int8 tensor of the output shape."""
        L = _lib.load()
        if x.ndim != 4 or x.shape[3] != self.ic:
            raise ValueError("expected NHWC with %d channels, got %s" % (self.ic, tuple(x.shape)))
        b, ih, iw, _ = x.shape
        oh, ow = self.out_shape(ih, iw)
        if _is_torch(x):
            import torch
            if x.dtype != torch.int8 or not x.is_cuda or not x.is_contiguous():
                raise ValueError("expected a contiguous CUDA int8 tensor")
            if out is None:
                out = torch.empty((b, oh, ow, self.oc), dtype=torch.int8, device=x.device)
            elif (out.dtype != torch.int8 or not out.is_cuda or not out.is_contiguous()
                  or out.numel() != b * oh * ow * self.oc):
                raise ValueError("out must be a contiguous CUDA int8 tensor with %d elements" % (b * oh * ow * self.oc))
            _lib.check(L.mi_conv_run(self._h, x.data_ptr(), b, ih, iw, out.data_ptr(), _stream()), "mi_conv_run")
            return out
        x = _host_i8(x)
        out = np.empty((b, oh, ow, self.oc), np.int8)
        _lib.check(L.mi_conv_run_host(self._h, x.ctypes.data, b, ih, iw, out.ctypes.data), "mi_conv_run_host")
        return out


class DynamicQuantKernel(_Handle):
    """Per-tensor DynamicQuant fp32 -> int8.  ``run`` returns (q, QuantParam) -- the QuantParam is what the
    reference kernel writes onto its output tensor."""
    _destroy = "mi_dynquant_destroy"

    def __init__(self, symmetric=False, device=0):
        super().__init__()
        L = _lib.init(device)
        _lib.check(L.mi_dynquant_create(1 if symmetric else 0, C.byref(self._h)), "mi_dynquant_create")
        self.last = None

    def run(self, x, fetch_params=True):
        L = _lib.load()
        p = _lib.DqParams()
        if _is_torch(x):
            import torch
            if x.dtype != torch.float32 or not x.is_cuda or not x.is_contiguous():
                raise ValueError("expected a contiguous CUDA float32 tensor")
            q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
            s = _stream()
            _lib.check(L.mi_dynquant_run(self._h, x.data_ptr(), x.numel(), q.data_ptr(), s), "mi_dynquant_run")
            if not fetch_params:
                return q, None
            _lib.check(L.mi_dynquant_get_params(self._h, s, C.byref(p)), "mi_dynquant_get_params")
        else:
            x = np.ascontiguousarray(x)
            if x.dtype != np.float32:
                raise TypeError("DynamicQuant needs a float32 input")  # dynamic_quant.cc:389-395
            q = np.empty(x.shape, np.int8)
            _lib.check(L.mi_dynquant_run_host(self._h, x.ctypes.data, x.size, q.ctypes.data, C.byref(p)),
                       "mi_dynquant_run_host")
        self.last = p
        return q, QuantParam(p.scale, p.zero_point)

    def device_params(self):
        return _lib.load().mi_dynquant_device_params(self._h)

    def run_rows(self, x):
        """Per-channel activation scales as the converter asks for them for a MatMul input (prefer_axes = every axis
        but the last): x [..., K] -> (q, [QuantParam per row]).  numpy in: host path, list of QuantParam out.
        CUDA tensor in: device path, returns (q, params) with params a CUDA uint8 tensor of `rows` parameter
        blocks to hand to MatmulDynamicInt8Kernel.run(..., row_params=params)."""
        L = _lib.load()
        unit = x.shape[-1]
        if _is_torch(x):
            import torch
            if x.dtype != torch.float32 or not x.is_cuda or not x.is_contiguous():
                raise ValueError("expected a contiguous CUDA float32 tensor")
            rows = x.numel() // unit
            q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
            params = torch.empty(rows * C.sizeof(_lib.DqParams), dtype=torch.uint8, device=x.device)
            _lib.check(L.mi_dynquant_run_segments(self._h, x.data_ptr(), rows, unit, q.data_ptr(), params.data_ptr(),
                                                  _stream()), "mi_dynquant_run_segments")
            return q, params
        x = np.ascontiguousarray(x)
        if x.dtype != np.float32:
            raise TypeError("DynamicQuant needs a float32 input")
        rows = x.size // unit
        q = np.empty(x.shape, np.int8)
        p = (_lib.DqParams * rows)()
        _lib.check(L.mi_dynquant_run_segments_host(self._h, x.ctypes.data, rows, unit, q.ctypes.data, p),
                   "mi_dynquant_run_segments_host")
        return q, [QuantParam(e.scale, e.zero_point) for e in p]


class MatmulDynamicInt8Kernel(_Handle):
    """Dynamic-quant MatMul: int8 activations (scale / zero point supplied at every run) x int8 weights -> fp32."""
    _destroy = "mi_dynmm_destroy"

    def __init__(self, weight, bias, weight_quant, transpose_b=True, act=ACT_NONE, device=0, packed_sdot=None,
                 weight_sums=None, decode_pack=True):
        """packed_sdot=(N, K): `weight` is the flat byte string a model converted for the ARM dot-product kernel
        carries (blocks of 16 channels x 4 K-bytes, RowMajor2Row4x16MajorInt8 / RowMajor2Col4x16MajorInt8) and
        weight_sums, if given, its int32 weight-sums tensor [round_up(N, 16)].  decode_pack=False skips the blocked
        second copy of the weights that serves 2..64 rows, and 65..128 against at most 4096 channels with K >= 1024 (MI_DYNMM_NO_DECODE_PACK)."""
        super().__init__()
        L = _lib.init(device)
        weight = _host_i8(weight)
        if packed_sdot is not None:
            self.n, self.k = int(packed_sdot[0]), int(packed_sdot[1])
            need = -(-self.n // 16) * 16 * -(-self.k // 4) * 4
            if weight.size != need:
                raise ValueError("a packed weight for N=%d, K=%d has %d bytes, got %d" % (self.n, self.k, need, weight.size))
        else:
            self.n, self.k = (weight.shape if transpose_b else weight.shape[::-1])
        if bias is not None:
            bias = np.ascontiguousarray(bias)
            if bias.dtype != np.float32:
                raise TypeError("dynamic MatMul needs a float32 bias")  # matmul_dynamic_int8.cc:48-51
            if bias.size != self.n:
                raise ValueError("bias has %d entries, expected %d" % (bias.size, self.n))
        nq, scales, zps = _quant_arrays(weight_quant)
        sums = None
        if weight_sums is not None:
            weight_sums = np.ascontiguousarray(weight_sums, dtype=np.int32)
            if packed_sdot is None or weight_sums.size < self.n:
                raise ValueError("weight_sums goes with a packed weight and holds at least N entries")
            sums = weight_sums.ctypes.data_as(C.POINTER(C.c_int32))
        d = _lib.DynmmDesc(self.k, self.n, 1 if transpose_b else 0, act, nq, scales, zps,
                           (_lib.DYNMM_WEIGHT_PACKED_SDOT if packed_sdot is not None else 0)
                           | (0 if decode_pack else _lib.DYNMM_NO_DECODE_PACK), sums)
        _lib.check(L.mi_dynmm_create(C.byref(d), weight.ctypes.data, None if bias is None else bias.ctypes.data,
                                     C.byref(self._h)), "mi_dynmm_create")

    def run(self, a, in_quant=None, params_dev=None, row_params=None):
        """in_quant: one QuantParam (per-tensor input) or a list with one per row (per-channel input; the zero point
        used is the first one, as in the reference).  Device path alternatives: params_dev (address of the block a
        DynamicQuantKernel.run left on the device) or row_params (the tensor DynamicQuantKernel.run_rows returned)."""
        L = _lib.load()
        if _is_torch(a):
            import torch
            if a.dtype != torch.int8 or not a.is_cuda or not a.is_contiguous() or a.shape[-1] != self.k:
                raise ValueError("expected a contiguous CUDA int8 tensor [..., %d]" % self.k)
            rows = a.numel() // self.k
            out = torch.empty(a.shape[:-1] + (self.n,), dtype=torch.float32, device=a.device)
            if row_params is not None:
                if row_params.numel() != rows * C.sizeof(_lib.DqParams):
                    raise ValueError("row_params does not hold %d parameter blocks" % rows)
                _lib.check(L.mi_dynmm_run_rows(self._h, a.data_ptr(), rows, row_params.data_ptr(), out.data_ptr(),
                                               _stream()), "mi_dynmm_run_rows")
            elif params_dev is not None:
                _lib.check(L.mi_dynmm_run_chained(self._h, a.data_ptr(), rows, params_dev, out.data_ptr(), _stream()),
                           "mi_dynmm_run_chained")
            else:
                _lib.check(L.mi_dynmm_run(self._h, a.data_ptr(), rows, float(in_quant.scale),
                                          int(in_quant.zero_point), out.data_ptr(), _stream()), "mi_dynmm_run")
            return out
        a = _host_i8(a)
        rows = a.size // self.k
        out = np.empty(a.shape[:-1] + (self.n,), np.float32)
        if not isinstance(in_quant, QuantParam):  # a sequence: one QuantParam per row
            in_quant = list(in_quant)
            if len(in_quant) != rows:
                raise ValueError("need one input QuantParam per row (%d), got %d" % (rows, len(in_quant)))
            scales = (C.c_double * rows)(*[float(qp.scale) for qp in in_quant])
            _lib.check(L.mi_dynmm_run_rows_host(self._h, a.ctypes.data, rows, scales, int(in_quant[0].zero_point),
                                                out.ctypes.data), "mi_dynmm_run_rows_host")
            return out
        _lib.check(L.mi_dynmm_run_host(self._h, a.ctypes.data, rows, float(in_quant.scale), int(in_quant.zero_point),
                                       out.ctypes.data), "mi_dynmm_run_host")
        return out


# ---- shape inference (host arithmetic; what a provider's KernelInterface::Infer answers) ----

def _shape_arg(shape):
    shape = [] if shape is None else [int(d) for d in shape]
    return (C.c_int32 * max(len(shape), 1))(*shape), len(shape)


def _shape_result(code, what, out, out_dims):
    _lib.check(code, what)
    return [out[i] for i in range(out_dims.value)]


def infer_matmul_shape(a_shape, b_shape, bias_shape=None, transpose_a=False, transpose_b=False):
    """Output shape of MatMulFusion as ``MatmulInferShape`` derives it; raises ``MiError`` with code -501 while an
    input dimension is unknown and -500 when the shapes do not fit."""
    L = _lib.load()
    a, an = _shape_arg(a_shape)
    b, bn = _shape_arg(b_shape)
    bias, biasn = _shape_arg(bias_shape)
    out, out_dims = (C.c_int32 * 8)(), C.c_int32(0)
    code = L.mi_infer_matmul(a, an, b, bn, bias, biasn, int(transpose_a), int(transpose_b), out, C.byref(out_dims))
    return _shape_result(code, "mi_infer_matmul", out, out_dims)


def infer_fullconnection_shape(a_shape, w_shape, bias_shape=None, has_bias=None, use_axis=False, axis=0):
    """Output shape of FullConnection as ``FullConnectionInferShape`` derives it."""
    L = _lib.load()
    a, an = _shape_arg(a_shape)
    w, wn = _shape_arg(w_shape)
    bias, biasn = _shape_arg(bias_shape)
    if has_bias is None:
        has_bias = bias_shape is not None
    out, out_dims = (C.c_int32 * 8)(), C.c_int32(0)
    code = L.mi_infer_fullconnection(a, an, w, wn, bias, biasn, int(has_bias), int(use_axis), int(axis), out,
                                     C.byref(out_dims))
    return _shape_result(code, "mi_infer_fullconnection", out, out_dims)


def infer_conv2d_shape(in_shape, w_shape, kernel=(-1, -1), stride=(1, 1), dilation=(1, 1), pad_mode=0,
                       pads=(0, 0, 0, 0), group=1):
    """Output shape of Conv2DFusion as ``Conv2dInferShape`` derives it, and the parameters it settles: returns
    ``(out_shape, (pad_u, pad_d, pad_l, pad_r), (kernel_h, kernel_w), group)``.  pad_mode: 0 explicit, 1 SAME,
    2 VALID."""
    L = _lib.load()
    x, xn = _shape_arg(in_shape)
    w, wn = _shape_arg(w_shape)
    p = _lib.ConvInfer(kernel[0], kernel[1], stride[0], stride[1], dilation[0], dilation[1], pad_mode,
                       pads[0], pads[1], pads[2], pads[3], group)
    out, out_dims = (C.c_int32 * 8)(), C.c_int32(0)
    code = L.mi_infer_conv2d(x, xn, w, wn, C.byref(p), out, C.byref(out_dims))
    shape = _shape_result(code, "mi_infer_conv2d", out, out_dims)
    return shape, (p.pad_u, p.pad_d, p.pad_l, p.pad_r), (p.kernel_h, p.kernel_w), p.group
