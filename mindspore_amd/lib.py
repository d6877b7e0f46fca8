"""ctypes binding of libmi355x_int8.so (the C ABI declared in include/mi355x_int8.h).

There is no CPU fallback: if the library is missing, or no gfx950 GPU is present when a kernel is created, the
call raises."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MI355X_INT8_LIB", os.path.join(HERE, "libmi355x_int8.so"))

MI_OK, MI_ERROR, MI_NULL_PTR, MI_PARAM_INVALID, MI_MEMORY_FAILED, MI_NOT_SUPPORT = 0, -1, -2, -3, -6, -7
ACT_NONE, ACT_RELU, ACT_RELU6 = 0, 1, 3

EXPORTS = [
    "mi_init", "mi_last_error", "mi_debug_fail_alloc", "mi_debug_sync_count", "mi_version", "mi_quantize_multiplier", "mi_quantize_multiplier_single", "mi_activation_range", "mi_requant_params",
    "mi_multiply_by_quantized_multiplier",
    "mi_matmul_create", "mi_matmul_reserve", "mi_matmul_run", "mi_matmul_run_noalloc", "mi_matmul_run_host", "mi_matmul_run_group", "mi_matmul_run_batched", "mi_matmul_broadcast_offsets", "mi_matmul_get_params", "mi_matmul_destroy",
    "mi_conv_create", "mi_conv_out_shape", "mi_conv_same_pad", "mi_conv_run", "mi_conv_run_host", "mi_conv_reserve", "mi_conv_destroy",
    "mi_dynquant_create", "mi_dynquant_run", "mi_dynquant_get_params", "mi_dynquant_device_params",
    "mi_dynquant_run_host", "mi_dynquant_run_segments", "mi_dynquant_run_segments_host", "mi_dynquant_destroy",
    "mi_unpack_weight_4x16", "mi_dynmm_create", "mi_dynmm_run", "mi_dynmm_run_chained", "mi_dynmm_run_host", "mi_dynmm_run_rows", "mi_dynmm_run_group", "mi_dynmm_run_rows_host", "mi_dynmm_reserve",
    "mi_dynmm_destroy",
    "mi_infer_matmul", "mi_infer_fullconnection", "mi_infer_conv2d",
    "mi_device_malloc", "mi_device_free", "mi_copy_to_device", "mi_copy_to_host", "mi_copy_to_host_async", "mi_stream_synchronize", "mi_stream_create", "mi_stream_destroy",
    "mi_host_malloc", "mi_host_free",
]
# libmi355x_diag.so (include/mi355x_diag.h): the benchmark's measurement aids, not part of the product library
DIAG_LIB_PATH = os.path.join(HERE, "libmi355x_diag.so")
DIAG_EXPORTS = ["mi_diag_stream_read", "mi_diag_copy", "mi_diag_mfma_rate"]


class MatmulDesc(C.Structure):
    _fields_ = [("deep", C.c_int32), ("col", C.c_int32), ("b_transpose", C.c_int32), ("act_type", C.c_int32),
                ("in_scale", C.c_double), ("in_zp", C.c_int32), ("out_scale", C.c_double), ("out_zp", C.c_int32),
                ("filter_quant_num", C.c_int32), ("filter_scales", C.POINTER(C.c_double)),
                ("filter_zps", C.POINTER(C.c_int32)), ("flags", C.c_int32), ("b_batch", C.c_int32)]


MATMUL_NO_DECODE_PACK = 1


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_channel", "out_channel", "kernel_h", "kernel_w", "stride_h", "stride_w", "dilation_h", "dilation_w",
        "pad_u", "pad_d", "pad_l", "pad_r", "group", "act_type")] + [
        ("in_scale", C.c_double), ("in_zp", C.c_int32), ("out_scale", C.c_double), ("out_zp", C.c_int32),
        ("filter_quant_num", C.c_int32), ("filter_scales", C.POINTER(C.c_double)),
        ("filter_zps", C.POINTER(C.c_int32)), ("flags", C.c_int32)]


CONV_3X3_EXACT = 1


class DynmmDesc(C.Structure):
    _fields_ = [("deep", C.c_int32), ("col", C.c_int32), ("b_transpose", C.c_int32), ("act_type", C.c_int32),
                ("filter_quant_num", C.c_int32), ("filter_scales", C.POINTER(C.c_double)),
                ("filter_zps", C.POINTER(C.c_int32)), ("flags", C.c_int32), ("weight_sums", C.POINTER(C.c_int32))]


DYNMM_WEIGHT_PACKED_SDOT = 1
DYNMM_NO_DECODE_PACK = 2


class ConvInfer(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "kernel_h", "kernel_w", "stride_h", "stride_w", "dilation_h", "dilation_w", "pad_mode",
        "pad_u", "pad_d", "pad_l", "pad_r", "group")]


class DqParams(C.Structure):
    _fields_ = [("scale", C.c_double), ("scale_f", C.c_float), ("zero_point", C.c_int32), ("real_min", C.c_float),
                ("real_max", C.c_float)]


class MiError(RuntimeError):
    def __init__(self, what, code, message):
        super().__init__("%s failed with status %d: %s" % (what, code, message))
        self.code = code


_lib = None
_initialised = False


def load():
    """Loads the shared library (no GPU needed for this step)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is not built: run `python -m mindspore_amd.build` (hipcc, gfx950)" % LIB_PATH)
    # A process must hold ONE HIP runtime.  PyTorch ships its own libamdhip64 (same SONAME as /opt/rocm's); when this
    # process is going to use torch for device memory and streams, torch's copy has to be the one that is loaded, so
    # import it before the dynamic loader resolves this library's dependency.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, i32, i64, dbl = C.c_void_p, C.c_int32, C.c_int64, C.c_double
    pi32 = C.POINTER(C.c_int32)
    L.mi_init.argtypes = [C.c_int]
    L.mi_last_error.restype = C.c_char_p
    L.mi_version.restype = C.c_char_p
    L.mi_quantize_multiplier.argtypes = [dbl, pi32, pi32, pi32]
    L.mi_quantize_multiplier_single.argtypes = [dbl, pi32, pi32, pi32]
    L.mi_activation_range.argtypes = [i32, i32, dbl, pi32, pi32]
    L.mi_requant_params.argtypes = [dbl, C.POINTER(dbl), i32, dbl, pi32, pi32, pi32]
    L.mi_multiply_by_quantized_multiplier.argtypes = [i32, i32, i32, i32]
    L.mi_multiply_by_quantized_multiplier.restype = i32
    L.mi_matmul_create.argtypes = [C.POINTER(MatmulDesc), vp, vp, C.POINTER(vp)]
    L.mi_matmul_reserve.argtypes = [vp, i32]
    L.mi_matmul_run.argtypes = [vp, vp, i32, vp, vp]
    L.mi_matmul_run_noalloc.argtypes = [vp, vp, i32, vp, vp]
    L.mi_matmul_run_group.argtypes = [C.POINTER(vp), i32, vp, i32, C.POINTER(vp), vp]
    L.mi_matmul_run_host.argtypes = [vp, vp, i32, vp]
    L.mi_matmul_run_batched.argtypes = [vp, vp, i32, i32, pi32, pi32, vp, vp]
    L.mi_matmul_broadcast_offsets.argtypes = [pi32, i32, pi32, i32, i32, pi32, pi32, pi32]
    L.mi_debug_fail_alloc.argtypes = [C.c_size_t]
    L.mi_matmul_get_params.argtypes = [vp, vp, vp, vp, vp, pi32, pi32]
    L.mi_matmul_destroy.argtypes = [vp]
    L.mi_matmul_destroy.restype = None
    L.mi_conv_create.argtypes = [C.POINTER(ConvDesc), vp, vp, C.POINTER(vp)]
    L.mi_conv_out_shape.argtypes = [vp, i32, i32, pi32, pi32]
    L.mi_conv_same_pad.argtypes = [i32, i32, i32, i32, pi32, pi32, pi32]
    L.mi_conv_run.argtypes = [vp, vp, i32, i32, i32, vp, vp]
    L.mi_conv_run_host.argtypes = [vp, vp, i32, i32, i32, vp]
    L.mi_conv_reserve.argtypes = [vp, i32, i32, i32]
    L.mi_conv_destroy.argtypes = [vp]
    L.mi_conv_destroy.restype = None
    L.mi_dynquant_create.argtypes = [i32, C.POINTER(vp)]
    L.mi_dynquant_run.argtypes = [vp, vp, i64, vp, vp]
    L.mi_dynquant_get_params.argtypes = [vp, vp, C.POINTER(DqParams)]
    L.mi_dynquant_device_params.argtypes = [vp]
    L.mi_dynquant_device_params.restype = vp
    L.mi_dynquant_run_host.argtypes = [vp, vp, i64, vp, C.POINTER(DqParams)]
    L.mi_dynquant_run_segments.argtypes = [vp, vp, i64, i64, vp, vp, vp]
    L.mi_dynquant_run_segments_host.argtypes = [vp, vp, i64, i64, vp, vp]
    L.mi_dynquant_destroy.argtypes = [vp]
    L.mi_dynquant_destroy.restype = None
    L.mi_unpack_weight_4x16.argtypes = [vp, i32, i32, vp]
    L.mi_dynmm_create.argtypes = [C.POINTER(DynmmDesc), vp, vp, C.POINTER(vp)]
    L.mi_dynmm_run.argtypes = [vp, vp, i32, dbl, i32, vp, vp]
    L.mi_dynmm_run_chained.argtypes = [vp, vp, i32, vp, vp, vp]
    L.mi_dynmm_run_host.argtypes = [vp, vp, i32, dbl, i32, vp]
    L.mi_dynmm_run_rows.argtypes = [vp, vp, i32, vp, vp, vp]
    L.mi_dynmm_run_group.argtypes = [C.POINTER(vp), i32, vp, i32, C.c_double, i32, vp, i32, C.POINTER(vp), vp]
    L.mi_dynmm_run_rows_host.argtypes = [vp, vp, i32, C.POINTER(dbl), i32, vp]
    L.mi_dynmm_reserve.argtypes = [vp, i32]
    L.mi_dynmm_destroy.argtypes = [vp]
    L.mi_dynmm_destroy.restype = None
    L.mi_infer_matmul.argtypes = [pi32, i32, pi32, i32, pi32, i32, i32, i32, pi32, pi32]
    L.mi_infer_fullconnection.argtypes = [pi32, i32, pi32, i32, pi32, i32, i32, i32, i32, pi32, pi32]
    L.mi_infer_conv2d.argtypes = [pi32, i32, pi32, i32, C.POINTER(ConvInfer), pi32, pi32]
    L.mi_device_malloc.argtypes = [C.c_size_t, C.POINTER(vp)]
    L.mi_device_free.argtypes = [vp]
    L.mi_host_malloc.argtypes = [C.c_size_t, C.POINTER(vp)]
    L.mi_host_free.argtypes = [vp]
    L.mi_copy_to_device.argtypes = [vp, vp, C.c_size_t, vp]
    L.mi_copy_to_host.argtypes = [vp, vp, C.c_size_t, vp]
    L.mi_copy_to_host_async.argtypes = [vp, vp, C.c_size_t, vp]
    L.mi_debug_sync_count.restype = C.c_int64
    L.mi_stream_synchronize.argtypes = [vp]
    L.mi_stream_create.argtypes = [C.POINTER(vp)]
    L.mi_stream_destroy.argtypes = [vp]
    _lib = L
    return L


_diag = None


def load_diag():
    """Loads the benchmark's measurement aids (libmi355x_diag.so)."""
    global _diag
    if _diag is not None:
        return _diag
    load()  # settles which HIP runtime the process holds
    if not os.path.exists(DIAG_LIB_PATH):
        raise RuntimeError("%s is not built: run `python -m mindspore_amd.build`" % DIAG_LIB_PATH)
    D = C.CDLL(DIAG_LIB_PATH)
    vp, i32, i64 = C.c_void_p, C.c_int32, C.c_int64
    D.mi_diag_stream_read.argtypes = [vp, i64, vp]
    D.mi_diag_copy.argtypes = [vp, vp, i64, vp]
    D.mi_diag_mfma_rate.argtypes = [vp, i32, i32, vp, vp]
    _diag = D
    return D


def check(code, what):
    if code != MI_OK:
        raise MiError(what, code, load().mi_last_error().decode())


def init(device=0):
    """Selects the GPU; raises if there is no gfx950 device."""
    global _initialised
    L = load()
    if not _initialised:
        check(L.mi_init(device), "mi_init")
        _initialised = True
    return L
