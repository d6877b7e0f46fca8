"""The MindSpore Lite provider (mindspore_amd/provider/mi355x_provider.cc) without a Lite SDK:
  * compiled against the reference's own public headers, with only the flatc-generated schema header replaced by a
    hand-written stand-in (CPU, needs the reference tree);
  * compiled against the stand-in Lite API of tests/lite_stub and driven by a harness that plays the scheduler:
    creator lookup by (arch, provider, data type, op type), shape inference, Prepare / ReSize / Execute.  On the CPU
    every creator must decline (no gfx950: the scheduler would fall back to the builtin kernels); on the GPU the outputs
    must equal the oracle's, as for the C ABI itself."""
import ctypes as C
import os

import numpy as np
import pytest

from tests.lite_stub import build as stub_build

I8, I32, F32 = 32, 34, 43
MATMUL, FC, CONV, DYNQUANT = 89, 67, 35, 203
OK, NO_CREATOR, DECLINED, INFER_FAILED, PREPARE_FAILED, RESIZE_FAILED, EXECUTE_FAILED, DECLINED_NO_FALLBACK = range(8)


class PhTensor(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("dims", C.c_int32), ("shape", C.c_int64 * 8), ("data", C.c_void_p),
                ("bytes", C.c_int64), ("is_const", C.c_int32), ("nquant", C.c_int32),
                ("scales", C.POINTER(C.c_double)), ("zps", C.POINTER(C.c_int32))]


class PhOp(C.Structure):
    _fields_ = [("type", C.c_int32), ("transpose_a", C.c_int32), ("transpose_b", C.c_int32), ("act", C.c_int32),
                ("has_bias", C.c_int32), ("use_axis", C.c_int32), ("axis", C.c_int32),
                ("kernel", C.c_int64 * 2), ("stride", C.c_int64 * 2), ("dilation", C.c_int64 * 2),
                ("pad_list", C.c_int64 * 4), ("has_pad_list", C.c_int32), ("pad_mode", C.c_int32),
                ("group", C.c_int64), ("in_channel", C.c_int64), ("out_channel", C.c_int64),
                ("symmetric", C.c_int32), ("dst_type", C.c_int64), ("n_prefer_axes", C.c_int32),
                ("prefer_axes", C.c_int32 * 8)]


def _load_harness():
    from mindspore_amd import lib
    lib.load()  # maps the HIP runtime and libmi355x_int8.so first
    if not os.path.exists(stub_build.OUT):
        stub_build.build_harness()
    h = C.CDLL(stub_build.OUT)
    h.ph_create.restype = C.c_void_p
    h.ph_create.argtypes = [C.POINTER(PhOp), C.c_char_p, C.c_char_p, C.POINTER(PhTensor), C.c_int32, C.c_int32,
                            C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_int32), C.POINTER(C.c_int32),
                            C.POINTER(C.c_int32)]
    h.ph_execute.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int32, C.c_int32,
                             C.POINTER(C.c_double), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    h.ph_output.restype = C.c_int64
    h.ph_output.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.c_void_p, C.c_int64,
                            C.POINTER(C.c_double), C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_int32)]
    h.ph_infer.argtypes = [C.POINTER(PhOp), C.c_char_p, C.POINTER(PhTensor), C.c_int32, C.POINTER(C.c_int64)]
    h.ph_destroy.argtypes = [C.c_void_p]
    h.ph_destroy.restype = None
    h.ph_create_node.restype = C.c_void_p
    h.ph_create_node.argtypes = h.ph_create.argtypes[:9] + [C.c_void_p, C.c_char_p, C.c_char_p] + h.ph_create.argtypes[9:]
    h.ph_execute_linked.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
    h.ph_resize_linked.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
    h.ph_set_enable_parallel.argtypes = [C.c_void_p, C.c_int32]
    h.ph_set_enable_parallel.restype = None
    h.mi355x_provider_group_launches.restype = C.c_int64
    h.ph_set_input_device_data.argtypes = [C.c_void_p, C.c_void_p]
    h.ph_set_input_device_data.restype = None
    h.ph_output_state.argtypes = [C.c_void_p]
    h.ph_has_provider_interface.argtypes = [C.c_char_p, C.c_int32]
    h.ph_register_test_interface.argtypes = [C.c_char_p, C.c_int32]
    h.ph_register_test_interface.restype = None
    h.ph_execute_concurrently.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]
    h.ph_lookup.argtypes = [C.c_char_p, C.c_char_p, C.c_int32, C.c_int32]
    h.ph_register_declining.argtypes = [C.c_char_p, C.c_char_p, C.c_int32, C.c_int32]
    return h


@pytest.fixture(scope="module")
def H():
    return _load_harness()


_keep = []  # ctypes buffers referenced by PhTensor structs


def tensor(dtype, shape, data=None, const=False, quant=()):
    t = PhTensor()
    t.dtype, t.dims, t.is_const = dtype, len(shape), int(const)
    for i, d in enumerate(shape):
        t.shape[i] = d
    if data is not None:
        data = np.ascontiguousarray(data)
        _keep.append(data)
        t.data, t.bytes = data.ctypes.data, data.nbytes
    scales = (C.c_double * max(len(quant), 1))(*[float(q[0]) for q in quant])
    zps = (C.c_int32 * max(len(quant), 1))(*[int(q[1]) for q in quant])
    _keep.extend([scales, zps])
    t.nquant, t.scales, t.zps = len(quant), scales, zps
    return t


def op(type_, **kw):
    o = PhOp()
    o.type = type_
    o.dst_type = I8
    o.group = 1
    for k, v in kw.items():
        if isinstance(v, (tuple, list)):
            arr = getattr(o, k)
            for i, x in enumerate(v):
                arr[i] = x
        else:
            setattr(o, k, v)
    return o


class Node:
    def __init__(self, H, o, inputs, out_dtype, out_quant=(), arch=b"CPU", provider=b"mi355x", producer=None,
                 out_name=None, device_only=None):
        """producer: the node whose output tensor is this node's input 0 (inputs[0] then only fills the slot);
        device_only: value of device_only_outputs in the [mi355x] section of the session config."""
        self.H = H
        arr = (PhTensor * len(inputs))(*inputs)
        scales = (C.c_double * max(len(out_quant), 1))(*[float(q[0]) for q in out_quant])
        zps = (C.c_int32 * max(len(out_quant), 1))(*[int(q[1]) for q in out_quant])
        stage, code = C.c_int32(-1), C.c_int32(0)
        self.h = H.ph_create_node(C.byref(o), arch, provider, arr, len(inputs), out_dtype, len(out_quant), scales, zps,
                                  producer.h if producer is not None else None, out_name, device_only,
                                  C.byref(stage), C.byref(code))
        self.stage, self.code, self.out_dtype = stage.value, code.value, out_dtype

    def run(self, x, quant=()):
        x = np.ascontiguousarray(x)
        shape = (C.c_int64 * x.ndim)(*x.shape)
        scales = (C.c_double * max(len(quant), 1))(*[float(q[0]) for q in quant])
        zps = (C.c_int32 * max(len(quant), 1))(*[int(q[1]) for q in quant])
        code = C.c_int32(0)
        st = self.H.ph_execute(self.h, x.ctypes.data, shape, x.ndim, len(quant), scales, zps, C.byref(code))
        assert st == OK, (st, code.value)
        return self.output()

    def run_linked(self):
        """Executes on the producer's output tensor as the producer left it."""
        code = C.c_int32(0)
        st = self.H.ph_execute_linked(self.h, C.byref(code))
        assert st == OK, (st, code.value)

    def resize_linked(self):
        """Shape inference and ReSize() on the producer's current output shape, without executing."""
        code = C.c_int32(0)
        st = self.H.ph_resize_linked(self.h, C.byref(code))
        assert st == OK, (st, code.value)

    def state(self):
        """(output has host memory, output carries a device address)"""
        st = self.H.ph_output_state(self.h)
        return bool(st & 1), bool(st & 2)

    def output(self):
        oshape, dims, nq = (C.c_int64 * 8)(), C.c_int32(0), C.c_int32(0)
        qs, qz = (C.c_double * 65536)(), (C.c_int32 * 65536)()
        nbytes = self.H.ph_output(self.h, oshape, C.byref(dims), None, 0, qs, qz, 65536, C.byref(nq))
        out = np.empty(nbytes, np.uint8)
        self.H.ph_output(self.h, oshape, C.byref(dims), out.ctypes.data, nbytes, qs, qz, 65536, C.byref(nq))
        np_dtype = {I8: np.int8, F32: np.float32}[self.out_dtype]
        y = out.view(np_dtype).reshape([oshape[i] for i in range(dims.value)])
        return y, [(qs[i], qz[i]) for i in range(nq.value)]

    def close(self):
        if self.h:
            self.H.ph_destroy(self.h)
            self.h = None


def _fc_inputs(rng, m, n, k, bias=True, w_const=True):
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    b = rng.integers(-5000, 5001, n).astype(np.int32) if bias else None
    ins = [tensor(I8, (m, k), None, False, [(0.02, -3)]),
           tensor(I8, (n, k), w, w_const, [(s, 0) for s in sw])]
    if bias:
        ins.append(tensor(I32, (n,), b, True))
    return a, w, sw, b, ins


# ---------------------------------------------------------------------------------------------------- CPU
def test_provider_compiles_against_reference_headers():
    out = stub_build.syntax_check_against_reference_headers()
    if out is None:
        pytest.skip("reference tree absent")
    assert out == "", out


def test_shape_inference_of_the_four_operators(H):
    """The provider registers no KernelInterface (the builtin inference keeps the nodes' OpParameters, see the next
    test); the harness's stand-in for the builtin inference runs on the library's mi_infer_* functions."""
    for t in (MATMUL, FC, CONV, DYNQUANT):
        assert H.ph_has_provider_interface(b"mi355x", t) == 0
    shp = (C.c_int64 * 8)()
    ins = (PhTensor * 2)(tensor(I8, (2, 5, 128), None), tensor(I8, (96, 128), None, True))
    assert H.ph_infer(C.byref(op(MATMUL, transpose_b=1)), b"mi355x", ins, 2, shp) == 3 and list(shp[:3]) == [2, 5, 96]
    assert H.ph_infer(C.byref(op(FC)), b"mi355x", ins, 2, shp) == 2 and list(shp[:2]) == [10, 96]
    ins = (PhTensor * 2)(tensor(I8, (1, 224, 224, 3), None), tensor(I8, (32, 3, 3, 3), None, True))
    conv = op(CONV, kernel=(3, 3), stride=(2, 2), dilation=(1, 1), pad_mode=1, in_channel=3, out_channel=32)
    assert H.ph_infer(C.byref(conv), b"mi355x", ins, 2, shp) == 4 and list(shp[:4]) == [1, 112, 112, 32]
    ins = (PhTensor * 2)(tensor(I8, (1, -1, 224, 3), None), tensor(I8, (32, 3, 3, 3), None, True))
    assert H.ph_infer(C.byref(conv), b"mi355x", ins, 2, shp) == -2          # unknown dimension: infer again later
    ins = (PhTensor * 2)(tensor(I8, (4, 7), None), tensor(I8, (96, 128), None, True))
    assert H.ph_infer(C.byref(op(MATMUL, transpose_b=1)), b"mi355x", ins, 2, shp) == -1
    ins = (PhTensor * 1)(tensor(F32, (3, 4, 5), None))
    assert H.ph_infer(C.byref(op(DYNQUANT)), b"mi355x", ins, 1, shp) == 3 and list(shp[:3]) == [3, 4, 5]
    # FullConnection with use_axis: the trailing axes fold into K
    ins = (PhTensor * 2)(tensor(I8, (2, 3, 4, 8), None), tensor(I8, (10, 32), None, True))
    assert H.ph_infer(C.byref(op(FC, use_axis=1, axis=2)), b"mi355x", ins, 2, shp) == 3 and list(shp[:3]) == [2, 3, 10]


def test_a_declined_node_can_still_fall_back(H):
    """Scheduler::InferNodeShape makes a node's OpParameter only when no provider KernelInterface answered for it
    (scheduler.cc:652-698), and the builtin kernel lookup needs that OpParameter (:1178-1183).  So a node that the
    provider declines must have been inferred by the builtin inference: the harness reports DECLINED then, and
    DECLINED_NO_FALLBACK when an interface registered under the provider's name has taken the inference over."""
    rng = np.random.default_rng(11)
    _, _, _, _, ins = _fc_inputs(rng, 4, 8, 16, w_const=False)   # a weight produced at run time: always declined
    node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)])
    assert node.stage == DECLINED and node.h is None
    fp32 = [tensor(F32, (4, 16), None), tensor(F32, (8, 16), rng.standard_normal((8, 16)).astype(np.float32), True)]
    assert Node(H, op(FC), fp32, F32).stage == NO_CREATOR        # fp32 nodes never reach this provider's creators
    # what registering an interface for a builtin operator would do (a provider name of the test's own, with the
    # mi355x creators behind it, is not available: the rule is shown on the real provider name, for MatMulFusion
    # only, and in a process of its own so that no other test sees the registration)
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r); import numpy as np; import tests.test_provider_harness as T;"
            "H = T._load_harness(); H.ph_register_test_interface(b'mi355x', T.MATMUL);"
            "rng = np.random.default_rng(3); ins = T._fc_inputs(rng, 4, 8, 16, bias=False, w_const=False)[4];"
            "n = T.Node(H, T.op(T.MATMUL, transpose_b=1), ins, T.I8, [(0.05, 5)]); print('stage', n.stage)"
            % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert "stage %d" % DECLINED_NO_FALLBACK in out.stdout, (out.stdout, out.stderr[-2000:])


def test_lookup_rules_of_the_kernel_registry(H):
    """The provider's registrations as the registry answers for them -- the reference's own RegisterKernel /
    RegistryKernelImpl (src/registry/register_kernel_impl.cc) when the harness was built with the reference tree at
    hand, the stand-in table otherwise: exact match on provider and arch (so the stock benchmark tool, which leaves
    the arch empty, needs the second registration), the data type of input 0 as part of the key, and at most ten
    providers per process."""
    real = bool(H.ph_registry_is_real())
    assert real == stub_build.real_registry_available() or not os.path.isdir(stub_build.REFERENCE)
    for arch in (b"CPU", b""):
        for dtype, ops in ((I8, (MATMUL, FC, CONV)), (F32, (DYNQUANT,))):
            for o in ops:
                assert H.ph_lookup(arch, b"mi355x", dtype, o) == 1, (arch, dtype, o)
    assert H.ph_lookup(b"GPU", b"mi355x", I8, MATMUL) == 0          # another arch
    assert H.ph_lookup(b"CPU", b"mi355", I8, MATMUL) == 0           # another provider name
    assert H.ph_lookup(b"CPU", b"", I8, MATMUL) == 0                # no provider: builtin kernels only
    assert H.ph_lookup(b"CPU", b"mi355x", F32, MATMUL) == 0         # fp32 MatMul is not this provider's
    assert H.ph_lookup(b"CPU", b"mi355x", I8, DYNQUANT) == 0        # DynamicQuant is keyed by its fp32 input
    assert H.ph_lookup(b"CPU", b"mi355x", I8, 36) == 0              # an operator type nobody registered
    if not real:
        return
    # register_kernel_impl.cc:32-36,105-117: op types outside (MIN, MAX] and data types outside the number range are
    # refused; an eleventh provider is refused (kMaxProviderNum = 10)
    assert H.ph_register_declining(b"CPU", b"probe0", I8, 0) != 0
    assert H.ph_register_declining(b"CPU", b"probe0", I8, 222) != 0
    assert H.ph_register_declining(b"CPU", b"probe0", 52, MATMUL) != 0
    assert H.ph_lookup(b"CPU", b"probe0", I8, MATMUL) == 0
    for i in range(9):  # mi355x is the first provider of the process
        assert H.ph_register_declining(b"CPU", b"probe%d" % i, I8, MATMUL) == 0, i
        assert H.ph_lookup(b"CPU", b"probe%d" % i, I8, MATMUL) == 1
    assert H.ph_register_declining(b"CPU", b"probe9", I8, MATMUL) != 0
    assert H.ph_lookup(b"CPU", b"probe9", I8, MATMUL) == 0
    assert H.ph_lookup(b"CPU", b"mi355x", I8, MATMUL) == 1          # the earlier registrations are untouched
    # a provider's eleventh arch is refused as well (kMaxArchPerProviderNum = 10); mi355x holds "CPU" and ""
    for i in range(8):
        assert H.ph_register_declining(b"arch%d" % i, b"mi355x", I8, 36) == 0, i
    assert H.ph_register_declining(b"arch8", b"mi355x", I8, 36) != 0


def test_registration_keys_and_decline_without_a_gpu(H):
    """Both arch keys are registered ("CPU" for applications, "" for the stock benchmark tool); an unknown key has no
    creator; without a gfx950 device every creator declines, so the scheduler would use the builtin kernels."""
    import torch
    rng = np.random.default_rng(0)
    a, w, sw, b, ins = _fc_inputs(rng, 4, 8, 16)
    node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], arch=b"GPU")
    assert node.stage == NO_CREATOR
    node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], provider=b"someone")
    assert node.stage == NO_CREATOR
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the creators accept")
    for arch in (b"CPU", b""):
        node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], arch=arch)
        assert node.stage == DECLINED and node.h is None


# ---------------------------------------------------------------------------------------------------- GPU
@pytest.mark.gpu
def test_fullconnection_and_matmul_through_the_provider(H, orc):
    rng = np.random.default_rng(1)
    for arch in (b"CPU", b""):
        a, w, sw, b, ins = _fc_inputs(rng, 128, 768, 768)
        node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], arch=arch)
        assert node.stage == OK, (node.stage, node.code)
        y, _ = node.run(a)
        want = orc.matmul_int8(a, w, b, 0.02, -3, sw, np.zeros(768, np.int32), 0.05, 5, 0, True)
        assert y.shape == (128, 768) and np.array_equal(y, want)
        # another row count through the same kernel: ReSize + Execute
        a2 = rng.integers(-128, 128, (5, 768), dtype=np.int8)
        y2, _ = node.run(a2)
        assert np.array_equal(y2, orc.matmul_int8(a2, w, b, 0.02, -3, sw, np.zeros(768, np.int32), 0.05, 5, 0, True))
        node.close()
    # MatMulFusion with a [K, N] weight, ReLU6, 3-D activation
    k, n = 100, 36
    a = rng.integers(-128, 128, (2, 7, k), dtype=np.int8)
    w = rng.integers(-128, 128, (k, n), dtype=np.int8)
    ins = [tensor(I8, a.shape, None, False, [(0.03, 4)]), tensor(I8, (k, n), w, True, [(0.004, 2)])]
    node = Node(H, op(MATMUL, transpose_b=0, act=3), ins, I8, [(0.04, -7)])
    assert node.stage == OK
    y, _ = node.run(a)
    want = orc.matmul_int8(a.reshape(14, k), w, None, 0.03, 4, np.array([0.004]), np.array([2], np.int32), 0.04, -7, 3,
                           False)
    assert y.shape == (2, 7, n) and np.array_equal(y.reshape(14, n), want)
    node.close()


@pytest.mark.gpu
@pytest.mark.parametrize("axis", [1, 2, 3])
def test_fullconnection_with_use_axis(H, orc, axis):
    """use_axis folds the input's axes from `axis` on into K: rows = product of the output's leading dimensions, K =
    the weight's second dimension (fullconnection_int8.cc:49-58)."""
    rng = np.random.default_rng(20 + axis)
    shape = (3, 4, 6, 8)
    k = int(np.prod(shape[axis:]))
    n = 40
    a = rng.integers(-128, 128, shape, dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    b = rng.integers(-5000, 5001, n).astype(np.int32)
    ins = [tensor(I8, shape, None, False, [(0.02, -3)]), tensor(I8, (n, k), w, True, [(s, 0) for s in sw]),
           tensor(I32, (n,), b, True)]
    node = Node(H, op(FC, has_bias=1, use_axis=1, axis=axis), ins, I8, [(0.05, 5)])
    assert node.stage == OK, (node.stage, node.code)
    y, _ = node.run(a)
    want = orc.matmul_int8(a.reshape(-1, k), w, b, 0.02, -3, sw, np.zeros(n, np.int32), 0.05, 5, 0, True)
    assert y.shape == shape[:axis] + (n,) and np.array_equal(y.reshape(-1, n), want)
    node.close()


@pytest.mark.gpu
def test_two_sessions_on_two_threads(H, orc):
    """Every session (Context) has a HIP stream of its own: two kernels of different sessions executed from two threads
    at the same time, 50 times each, both give the oracle's result."""
    rng = np.random.default_rng(31)
    a1, w1, sw1, b1, ins1 = _fc_inputs(rng, 96, 512, 1024)
    n1 = Node(H, op(FC, has_bias=1), ins1, I8, [(0.05, 5)])
    x = rng.integers(-128, 128, (2, 40, 40, 32), dtype=np.int8)
    wc = rng.integers(-128, 128, (48, 1, 1, 32), dtype=np.int8)
    swc = rng.uniform(1e-3, 1e-2, 48).astype(np.float32).astype(np.float64)
    conv = op(CONV, kernel=(1, 1), stride=(1, 1), dilation=(1, 1), pad_mode=2, in_channel=32, out_channel=48)
    n2 = Node(H, conv, [tensor(I8, x.shape, None, False, [(0.02, 1)]), tensor(I8, wc.shape, wc, True, [(s, 0) for s in swc])],
              I8, [(0.05, -2)])
    assert n1.stage == OK and n2.stage == OK, (n1.stage, n1.code, n2.stage, n2.code)
    want1 = orc.matmul_int8(a1, w1, b1, 0.02, -3, sw1, np.zeros(512, np.int32), 0.05, 5, 0, True)
    y1, _ = n1.run(a1)   # first runs: shapes set, outputs allocated
    y2, _ = n2.run(x)
    assert np.array_equal(y1, want1)
    a1b = np.ascontiguousarray(a1[::-1])
    xb = np.ascontiguousarray(x[:, ::-1])
    want2b, _ = n2.run(xb)
    assert H.ph_execute_concurrently(n1.h, a1b.ctypes.data, n2.h, x.ctypes.data, 50) == 0
    y1c, _ = n1.output()
    y2c, _ = n2.output()
    assert np.array_equal(y1c, orc.matmul_int8(a1b, w1, b1, 0.02, -3, sw1, np.zeros(512, np.int32), 0.05, 5, 0, True))
    assert np.array_equal(y2c, y2) and not np.array_equal(y2c, want2b)
    n1.close()
    n2.close()


@pytest.mark.gpu
def test_sibling_fullconnections_run_as_one_launch(H, orc):
    """Three FullConnection nodes of one session read the same tensor (the output of a fourth): the first one executed
    runs all three as one launch and the others deliver what it left; every output equals the oracle's, also after
    resizes, and beyond 32 rows every node runs by itself.  A session that executes its nodes in parallel forms no
    groups."""
    rng = np.random.default_rng(21)
    k0, k = 192, 512

    def fc(n, kk, producer=None, out_name=None):
        a, w, sw, b, ins = _fc_inputs(rng, 4, n, kk)
        ins[0] = tensor(I8, (4, kk), None, False, [(0.05, 5)]) if producer is not None else ins[0]
        node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], producer=producer, out_name=out_name)
        assert node.stage == OK, (node.stage, node.code)
        return node, w, sw, b

    for parallel in (False, True):
        head, w0, sw0, b0 = fc(k, k0, out_name=b"hidden")
        if parallel:
            H.ph_set_enable_parallel(head.h, 1)
        sibs = [fc(n, k, producer=head) for n in (384, 640, 96)]
        before = H.mi355x_provider_group_launches()
        runs = 0
        for rows in (4, 1, 7, 40):
            x = rng.integers(-128, 128, (rows, k0), dtype=np.int8)
            hidden, _ = head.run(x)
            want_h = orc.matmul_int8(x, w0, b0, 0.02, -3, sw0, np.zeros(k, np.int32), 0.05, 5, 0, True)
            assert np.array_equal(hidden, want_h)
            for node, *_ in sibs:  # the runtime resizes every node of the graph before it executes any
                node.resize_linked()
            for node, w, sw, b in sibs:
                node.run_linked()
                got, _ = node.output()
                want = orc.matmul_int8(want_h, w, b, 0.05, 5, sw, np.zeros(w.shape[0], np.int32), 0.05, 5, 0, True)
                assert got.shape == want.shape and np.array_equal(got, want), (parallel, rows, w.shape)
            runs += 1 if rows <= 32 else 0
        launches = H.mi355x_provider_group_launches() - before
        assert launches == (0 if parallel else runs), (parallel, launches)
        for node, *_ in reversed(sibs):
            node.close()
        head.close()


@pytest.mark.gpu
def test_a_sibling_result_is_not_delivered_for_a_later_version_of_the_input(H, orc):
    """Two siblings behind a provider kernel.  Run 1 executes only the first sibling, which launches for both; run 2
    (new input, same tensor memory) executes only the second: it must not hand out what run 1 left in its buffer.
    The producer counts its deliveries, and the second sibling sees that the count moved on."""
    rng = np.random.default_rng(23)
    k0, k = 96, 256

    def fc(n, kk, producer=None):
        a, w, sw, b, ins = _fc_inputs(rng, 4, n, kk)
        ins[0] = tensor(I8, (4, kk), None, False, [(0.05, 5)]) if producer is not None else ins[0]
        node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)], producer=producer)
        assert node.stage == OK, (node.stage, node.code)
        return node, w, sw, b

    head, w0, sw0, b0 = fc(k, k0)
    (first, w1, s1, b1), (second, w2, s2, b2) = fc(128, k, head), fc(64, k, head)
    before = H.mi355x_provider_group_launches()
    x1 = rng.integers(-128, 128, (4, k0), dtype=np.int8)
    h1, _ = head.run(x1)
    first.run_linked()   # launches for both siblings; the second one is not executed in this run
    assert H.mi355x_provider_group_launches() == before + 1
    x2 = rng.integers(-128, 128, (4, k0), dtype=np.int8)
    h2, _ = head.run(x2)
    assert not np.array_equal(h1, h2)
    second.run_linked()  # first in this run: computes from the new input
    got, _ = second.output()
    want = orc.matmul_int8(h2, w2, b2, 0.05, 5, s2, np.zeros(64, np.int32), 0.05, 5, 0, True)
    assert np.array_equal(got, want)
    first.run_linked()
    got, _ = first.output()
    assert np.array_equal(got, orc.matmul_int8(h2, w1, b1, 0.05, 5, s1, np.zeros(128, np.int32), 0.05, 5, 0, True))
    for node in (second, first, head):
        node.close()


@pytest.mark.gpu
def test_what_the_provider_declines(H):
    rng = np.random.default_rng(2)
    a, w, sw, b, ins = _fc_inputs(rng, 4, 8, 16, w_const=False)            # weight produced at run time
    assert Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)]).stage == DECLINED
    a, w, sw, b, ins = _fc_inputs(rng, 4, 8, 16)
    assert Node(H, op(MATMUL, transpose_a=1, transpose_b=1), ins, I8, [(0.05, 5)]).stage in (DECLINED, INFER_FAILED)
    assert Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5), (0.06, 5)]).stage == DECLINED   # per-channel output
    x = tensor(I8, (1, 8, 8, 4), None, False, [(0.02, 1)])
    wc = tensor(I8, (8, 3, 3, 4), rng.integers(-128, 128, (8, 3, 3, 4), dtype=np.int8), True, [(0.01, 0)])
    conv = op(CONV, kernel=(3, 3), stride=(1, 1), dilation=(1, 1), pad_mode=1, in_channel=4, out_channel=8)
    assert Node(H, conv, [x, wc], I8, [(0.05, 0)]).stage == DECLINED       # dense 3x3 stride 1: Winograd on the CPU
    dq = op(DYNQUANT, n_prefer_axes=1, prefer_axes=(1,))
    assert Node(H, dq, [tensor(F32, (4, 6, 8), None)], I8).stage == DECLINED  # would need the transposition


@pytest.mark.gpu
def test_conv_through_the_provider_with_resize(H, orc):
    from oracle.pyoracle import conv_shape
    rng = np.random.default_rng(3)
    ic, oc = 3, 32
    w = rng.integers(-128, 128, (oc, 3, 3, ic), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, oc).astype(np.float32).astype(np.float64)
    bias = rng.integers(-3000, 3001, oc).astype(np.int32)
    conv = op(CONV, kernel=(3, 3), stride=(2, 2), dilation=(1, 1), pad_mode=1, in_channel=ic, out_channel=oc, act=3)
    ins = [tensor(I8, (1, 224, 224, ic), None, False, [(0.02, 3)]), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
           tensor(I32, (oc,), bias, True)]
    node = Node(H, conv, ins, I8, [(0.03, -10)])
    assert node.stage == OK, (node.stage, node.code)
    for b, ih, iw, pad in [(1, 224, 224, (0, 1, 0, 1)), (2, 33, 17, (1, 1, 1, 1)), (1, 224, 224, (0, 1, 0, 1))]:
        x = rng.integers(-128, 128, (b, ih, iw, ic), dtype=np.int8)
        y, _ = node.run(x)          # SAME padding moves with the image size: ReSize rebuilds the handle
        shape = conv_shape(b, ih, iw, ic, oc, (3, 3), (2, 2), (1, 1), pad)
        want = orc.conv_int8(x, w, bias, shape, 0.02, 3, sw, np.zeros(oc, np.int32), 0.03, -10, 3)
        assert y.shape == want.shape and np.array_equal(y, want), (b, ih, iw)
    node.close()
    # depthwise 3x3 and a 1x1 with explicit padding
    c = 16
    wd = rng.integers(-128, 128, (c, 3, 3, 1), dtype=np.int8)
    swd = rng.uniform(1e-3, 1e-2, c).astype(np.float32).astype(np.float64)
    dw = op(CONV, kernel=(3, 3), stride=(1, 1), dilation=(1, 1), pad_mode=0, pad_list=(1, 1, 1, 1), has_pad_list=1,
            group=c, in_channel=c, out_channel=c)
    node = Node(H, dw, [tensor(I8, (1, 12, 12, c), None, False, [(0.02, -4)]),
                        tensor(I8, wd.shape, wd, True, [(s, 0) for s in swd])], I8, [(0.01, 2)])
    assert node.stage == OK, (node.stage, node.code)
    x = rng.integers(-128, 128, (1, 12, 12, c), dtype=np.int8)
    y, _ = node.run(x)
    shape = conv_shape(1, 12, 12, c, c, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1))
    want = orc.conv_dw_int8(x, wd.reshape(c, 3, 3), None, shape, 0.02, -4, swd, np.zeros(c, np.int32), 0.01, 2, 0)
    assert np.array_equal(y, want)
    node.close()


@pytest.mark.gpu
def test_dynamic_quant_and_dynamic_matmul_through_the_provider(H, orc):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((37, 96)) * 2).astype(np.float32)
    w = rng.integers(-127, 128, (80, 96), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, 80).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(80).astype(np.float32)
    zw = np.zeros(80, np.int32)
    mm_ins = lambda: [tensor(I8, (37, 96), None), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
                      tensor(F32, (80,), bias, True)]
    # per tensor: DynamicQuant writes {scale, zero point} onto its output tensor; the MatMul reads them at Execute
    dq = Node(H, op(DYNQUANT), [tensor(F32, x.shape, None)], I8)
    assert dq.stage == OK, (dq.stage, dq.code)
    q, qp = dq.run(x)
    q_ref, s_ref, z_ref = orc.dynamic_quant(x, False)
    assert np.array_equal(q, q_ref) and qp == [(s_ref, z_ref)]
    mm = Node(H, op(MATMUL, transpose_b=1), mm_ins(), F32)
    assert mm.stage == OK, (mm.stage, mm.code)
    y, _ = mm.run(q, qp)
    want = orc.dynamic_matmul(q_ref, w, bias, s_ref, z_ref, sw, zw)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    # per row (prefer_axes = the leading axis), symmetric as the converter emits it
    dqr = Node(H, op(DYNQUANT, symmetric=1, n_prefer_axes=1, prefer_axes=(0,)), [tensor(F32, x.shape, None)], I8)
    assert dqr.stage == OK, (dqr.stage, dqr.code)
    qr, qpr = dqr.run(x)
    qr_ref, scales_ref, zps_ref = orc.dynamic_quant_segments(x, True)
    assert np.array_equal(qr, qr_ref) and [p[0] for p in qpr] == list(scales_ref) and all(p[1] == 0 for p in qpr)
    yr, _ = mm.run(qr, qpr)
    wantr = orc.dynamic_matmul_rows(qr_ref, w, bias, scales_ref, 0, sw, zw)
    assert np.array_equal(yr.view(np.uint32), wantr.view(np.uint32))
    for n in (dq, mm, dqr):
        n.close()


@pytest.mark.gpu
def test_configuration_2_block_through_the_provider(H, orc):
    """The MobileNetV2-style block of benchmark configuration 2 (3x3 s2 stem, 1x1 expand, 3x3 depthwise, 1x1 project,
    ReLU6 fused) as four provider kernels in a row, tensors handed over on the host as a "CPU"-arch provider gets
    them: every layer's output equals the oracle's, and the last one the committed golden hash."""
    import hashlib
    import json
    from mindspore_amd import workloads as wl
    from oracle.pyoracle import conv_shape
    hashes = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "config_hashes.json")))["c2"]
    orc.set_threads(16)
    x, layers = wl.mobilenet_c2()
    cur = x
    for L in layers:
        dw = L["kind"] == "dw"
        w = L["w"].reshape(L["oc"], L["kernel"], L["kernel"], 1) if dw else L["w"]
        node_op = op(CONV, kernel=(L["kernel"],) * 2, stride=(L["stride"],) * 2, dilation=(1, 1), pad_mode=0,
                     pad_list=L["pad"], has_pad_list=1, group=L["oc"] if dw else 1, in_channel=L["ic"],
                     out_channel=L["oc"], act=L["act"])
        ins = [tensor(I8, cur.shape, None, False, [(L["sx"], L["zx"])]),
               tensor(I8, w.shape, w, True, [(s, z) for s, z in zip(L["sw"], L["zw"])])]
        if L["bias"] is not None:
            ins.append(tensor(I32, (L["oc"],), L["bias"], True))
        node = Node(H, node_op, ins, I8, [(L["so"], L["zo"])])
        assert node.stage == OK, (L["name"], node.stage, node.code)
        got, _ = node.run(cur)
        shape = conv_shape(cur.shape[0], cur.shape[1], cur.shape[2], L["ic"], L["oc"], (L["kernel"],) * 2,
                           (L["stride"],) * 2, (1, 1), L["pad"])
        fn = orc.conv_dw_int8 if dw else orc.conv_int8
        want = fn(cur, L["w"], L["bias"], shape, L["sx"], L["zx"], L["sw"], L["zw"], L["so"], L["zo"], L["act"])
        assert got.shape == want.shape and np.array_equal(got, want), L["name"]
        assert hashlib.sha256(np.ascontiguousarray(got).tobytes()).hexdigest() == hashes[L["name"]], L["name"]
        node.close()
        cur = got


def _c2_nodes(H, x_shape, layers, device_only):
    """The four convolutions as a graph: each node's input 0 is the tensor the node before wrote."""
    from oracle.pyoracle import conv_shape
    nodes, shape = [], x_shape
    for i, L in enumerate(layers):
        dw = L["kind"] == "dw"
        w = L["w"].reshape(L["oc"], L["kernel"], L["kernel"], 1) if dw else L["w"]
        node_op = op(CONV, kernel=(L["kernel"],) * 2, stride=(L["stride"],) * 2, dilation=(1, 1), pad_mode=0,
                     pad_list=L["pad"], has_pad_list=1, group=L["oc"] if dw else 1, in_channel=L["ic"],
                     out_channel=L["oc"], act=L["act"])
        ins = [tensor(I8, shape, None, False, [(L["sx"], L["zx"])]),
               tensor(I8, w.shape, w, True, [(s, z) for s, z in zip(L["sw"], L["zw"])]),
               tensor(I32, (L["oc"],), L["bias"], True)]
        node = Node(H, node_op, ins, I8, [(L["so"], L["zo"])], producer=nodes[-1] if nodes else None,
                    out_name=L["name"].encode(), device_only=device_only)
        assert node.stage == OK, (L["name"], node.stage, node.code)
        nodes.append(node)
        g = conv_shape(shape[0], shape[1], shape[2], L["ic"], L["oc"], (L["kernel"],) * 2, (L["stride"],) * 2, (1, 1),
                       L["pad"])
        shape = (g.batch, g.out_h, g.out_w, L["oc"])
    return nodes


def _c2_oracle(orc, x, layers):
    from oracle.pyoracle import conv_shape
    outs, cur = [], x
    for L in layers:
        shape = conv_shape(cur.shape[0], cur.shape[1], cur.shape[2], L["ic"], L["oc"], (L["kernel"],) * 2,
                           (L["stride"],) * 2, (1, 1), L["pad"])
        fn = orc.conv_dw_int8 if L["kind"] == "dw" else orc.conv_int8
        cur = fn(cur, L["w"], L["bias"], shape, L["sx"], L["zx"], L["sw"], L["zw"], L["so"], L["zo"], L["act"])
        outs.append(cur)
    return outs


@pytest.mark.gpu
def test_activations_stay_on_the_device_between_provider_kernels(H, orc):
    """Configuration 2 as a graph of four provider kernels whose intermediate tensors are shared objects.  By default
    every kernel publishes its device buffer on the output tensor and also fills the host copy; the next kernel reads
    the device buffer in place.  With the interior outputs declared device-only the host copies never come into being
    and only the last output travels back.  Both ways, run twice (second time on another image, of another size):
    every host-visible output equals the oracle's, the first image's last output the committed golden hash."""
    import hashlib
    import json
    from mindspore_amd import workloads as wl
    hashes = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "config_hashes.json")))["c2"]
    orc.set_threads(16)
    x, layers = wl.mobilenet_c2()
    x2 = np.random.default_rng(9).integers(-128, 128, (2, 97, 61, 3), dtype=np.int8)
    want = {0: _c2_oracle(orc, x, layers), 1: _c2_oracle(orc, x2, layers)}
    for device_only in (None, b"stem, expand,dw", b"*"):
        nodes = _c2_nodes(H, x.shape, layers, device_only)
        for which, image in ((0, x), (1, x2), (0, x)):
            nodes[0].run(image)
            for node in nodes[1:]:
                node.run_linked()
            for i, node in enumerate(nodes):
                host, dev = node.state()
                interior = i + 1 < len(nodes)
                assert dev, (device_only, i)
                if device_only is None:
                    assert host
                    got, _ = node.output()
                    assert got.shape == want[which][i].shape and np.array_equal(got, want[which][i]), (which, i)
                elif interior or device_only == b"*":
                    assert not host, (device_only, i)  # never allocated: nothing was copied back
            if device_only != b"*":
                got, _ = nodes[-1].output()
                assert np.array_equal(got, want[which][-1]), (device_only, which)
                if which == 0:
                    assert hashlib.sha256(np.ascontiguousarray(got).tobytes()).hexdigest() == hashes["project"]
        for node in reversed(nodes):
            node.close()


@pytest.mark.gpu
def test_dynamic_quant_feeds_the_dynamic_matmul_on_the_device(H, orc):
    """DynamicQuant -> dynamic MatMul sharing the int8 tensor.  The MatMul takes the bytes AND the scale / zero point
    (one block, or one per row) from device memory, where the DynamicQuant kernel of this provider left them.  By
    default the quant parameters also reach the host tensor (a builtin consumer would read them there); with the
    tensor declared device-only nothing travels to the host and nothing is waited for."""
    from mindspore_amd import lib
    L = lib.load()
    rng = np.random.default_rng(14)
    w = rng.integers(-127, 128, (80, 96), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, 80).astype(np.float32).astype(np.float64)
    bias = rng.standard_normal(80).astype(np.float32)
    zw = np.zeros(80, np.int32)
    for per_row in (False, True):
        for device_only in (None, b"q", b"*"):
            dq_op = op(DYNQUANT, symmetric=1, n_prefer_axes=1, prefer_axes=(0,)) if per_row else op(DYNQUANT)
            dq = Node(H, dq_op, [tensor(F32, (37, 96), None)], I8, out_name=b"q", device_only=device_only)
            assert dq.stage == OK, (dq.stage, dq.code)
            mm = Node(H, op(MATMUL, transpose_b=1),
                      [tensor(I8, (37, 96), None), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
                       tensor(F32, (80,), bias, True)], F32, producer=dq, out_name=b"y", device_only=device_only)
            assert mm.stage == OK, (mm.stage, mm.code)
            for rows in (37, 5, 64):
                x = (rng.standard_normal((rows, 96)) * 3).astype(np.float32)
                syncs0 = L.mi_debug_sync_count()
                _, qp = dq.run(x)
                syncs1 = L.mi_debug_sync_count()
                mm.run_linked()
                syncs2 = L.mi_debug_sync_count()
                if per_row:
                    q_ref, scales_ref, _ = orc.dynamic_quant_segments(x, True)
                    ref = orc.dynamic_matmul_rows(q_ref, w, bias, scales_ref, 0, sw, zw)
                    qp_ref = [(sc, 0) for sc in scales_ref]
                else:
                    q_ref, s_ref, z_ref = orc.dynamic_quant(x, False)
                    ref = orc.dynamic_matmul(q_ref, w, bias, s_ref, z_ref, sw, zw)
                    qp_ref = [(s_ref, z_ref)]
                if device_only is None:
                    # upload of x, then ONE wait for both the int8 bytes and the parameters; upload-free MatMul, one
                    # wait for its output
                    assert dq.state() == (True, True) and qp == qp_ref
                    assert (syncs1 - syncs0, syncs2 - syncs1) == (2, 1)
                else:
                    assert dq.state() == (False, True)
                    # after the upload of x the host waits for nothing until an output has to reach it
                    assert syncs1 - syncs0 == 1
                    assert syncs2 - syncs1 == (1 if device_only == b"q" else 0)
                if device_only != b"*":
                    y, _ = mm.output()
                    assert y.shape == ref.shape and np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (per_row, rows)
            mm.close()
            dq.close()


@pytest.mark.gpu
def test_sibling_dynamic_matmuls_run_as_one_launch(H, orc):
    """DynamicQuant feeding three dynamic MatMuls (q / k / v): at up to 32 rows the first MatMul executed runs all three
    as one launch, reading the scale where DynamicQuant left it on the device (one for the tensor, or one per row), and
    the others deliver what it left; beyond 32 rows every node runs by itself.  Every output equals the oracle's."""
    rng = np.random.default_rng(31)
    k = 256
    for per_row in (False, True):
        dq_op = op(DYNQUANT, symmetric=1, n_prefer_axes=1, prefer_axes=(0,)) if per_row else op(DYNQUANT)
        dq = Node(H, dq_op, [tensor(F32, (4, k), None)], I8, out_name=b"q")
        assert dq.stage == OK, (dq.stage, dq.code)
        sibs = []
        for n in (96, 320, 48):
            w = rng.integers(-127, 128, (n, k), dtype=np.int8)
            sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
            bias = rng.standard_normal(n).astype(np.float32)
            mm = Node(H, op(MATMUL, transpose_b=1),
                      [tensor(I8, (4, k), None), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
                       tensor(F32, (n,), bias, True)], F32, producer=dq)
            assert mm.stage == OK, (mm.stage, mm.code)
            sibs.append((mm, w, sw, bias))
        before = H.mi355x_provider_group_launches()
        runs = 0
        for rows in (4, 1, 9, 40):
            x = (rng.standard_normal((rows, k)) * 3).astype(np.float32)
            dq.run(x)
            for mm, *_ in sibs:
                mm.resize_linked()
            if per_row:
                q_ref, scales_ref, _ = orc.dynamic_quant_segments(x, True)
            else:
                q_ref, s_ref, z_ref = orc.dynamic_quant(x, False)
            for mm, w, sw, bias in sibs:
                mm.run_linked()
                y, _ = mm.output()
                zw = np.zeros(w.shape[0], np.int32)
                ref = orc.dynamic_matmul_rows(q_ref, w, bias, scales_ref, 0, sw, zw) if per_row else \
                    orc.dynamic_matmul(q_ref, w, bias, s_ref, z_ref, sw, zw)
                assert y.shape == ref.shape and np.array_equal(y.view(np.uint32), ref.view(np.uint32)), (per_row, rows)
            runs += 1 if rows <= 32 else 0
        assert H.mi355x_provider_group_launches() - before == runs, (per_row, runs)
        for mm, *_ in reversed(sibs):
            mm.close()
        dq.close()


@pytest.mark.gpu
def test_time_of_dynamic_quant_into_the_qkv_matmul(H, orc):
    """Per-layer host time of DynamicQuant (4096 x 768) -> QKV dynamic MatMul (2304 channels) through the provider:
    with every tensor handed over on the host, with the int8 tensor device-only, and with both outputs device-only
    (the part a following provider kernel would see).  Printed (-s shows it); the one assertion is that keeping the
    tensors on the device is not slower than copying them."""
    import time
    from mindspore_amd import lib, workloads as wl
    L = lib.load()
    x = wl.bert_c3_activation(768)
    wt = wl.bert_c3_weights("qkv", 2304, 768)
    times = {}
    for device_only in (None, b"q", b"*"):
        dq = Node(H, op(DYNQUANT), [tensor(F32, x.shape, None)], I8, out_name=b"q", device_only=device_only)
        mm = Node(H, op(MATMUL, transpose_b=1),
                  [tensor(I8, x.shape, None), tensor(I8, wt["w"].shape, wt["w"], True, [(s, 0) for s in wt["sw"]]),
                   tensor(F32, (2304,), wt["bias"], True)], F32, producer=dq, out_name=b"y", device_only=device_only)
        assert dq.stage == OK and mm.stage == OK
        for _ in range(3):
            dq.run(x)
            mm.run_linked()
        L.mi_stream_synchronize(None)
        syncs = L.mi_debug_sync_count()
        t0 = time.perf_counter()
        reps = 10
        for _ in range(reps):
            dq.run(x)
            mm.run_linked()
        L.mi_device_free(None)  # (no-op)
        t = (time.perf_counter() - t0) / reps
        times[device_only] = (t, (L.mi_debug_sync_count() - syncs) / reps)
        mm.close()
        dq.close()
    print("DynamicQuant -> QKV per layer (host clock, incl. the harness's copy of x into the input tensor): "
          + ", ".join("%s: %.0f us, %.0f waits" % (k.decode() if k else "host hand-over", v[0] * 1e6, v[1])
                      for k, v in times.items()))
    assert times[b"*"][0] <= times[None][0]


@pytest.mark.gpu
def test_batched_constant_weight_through_the_provider(H, orc):
    """MatMulFusion whose constant weight has rank 3: one output matrix per (activation matrix, weight matrix) pair
    by the reference's broadcast rule; the creator declines the same weight for FullConnection and for fp32 output."""
    from oracle import pyoracle
    rng = np.random.default_rng(21)
    n, k = 44, 80
    sw = rng.uniform(1e-3, 1e-2, n).astype(np.float32).astype(np.float64)
    bias = rng.integers(-3000, 3001, n).astype(np.int32)
    for a_shape, w_batch in (((3, 9, k), (3,)), ((2, 3, 40, k), (3,)), ((6, 5, k), (2,)), ((50, k), (4,))):
        w = rng.integers(-128, 128, w_batch + (n, k), dtype=np.int8)
        ins = [tensor(I8, a_shape, None, False, [(0.02, -3)]), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
               tensor(I32, (n,), bias, True)]
        node = Node(H, op(MATMUL, transpose_b=1), ins, I8, [(0.05, 5)])
        assert node.stage == OK, (node.stage, node.code)
        a = rng.integers(-128, 128, a_shape, dtype=np.int8)
        got, _ = node.run(a)
        a_off, b_off = pyoracle.broadcast_offsets(a_shape, w.shape)
        rows = a_shape[-2]
        assert got.size == len(a_off) * rows * n
        got = got.reshape(len(a_off), rows, n)
        for i, (ai, bi) in enumerate(zip(a_off, b_off)):
            want = orc.matmul_int8(a.reshape(-1, rows, k)[ai], w.reshape(-1, n, k)[bi], bias, 0.02, -3, sw,
                                   np.zeros(n, np.int32), 0.05, 5, 0, True)
            assert np.array_equal(got[i], want), (a_shape, w_batch, i)
        node.close()
    w = rng.integers(-128, 128, (3, n, k), dtype=np.int8)
    wq = [(s, 0) for s in sw]
    fc = Node(H, op(FC, has_bias=0), [tensor(I8, (3, 9, k), None, False, [(0.02, -3)]), tensor(I8, w.shape, w, True, wq)],
              I8, [(0.05, 5)])
    assert fc.stage in (DECLINED, INFER_FAILED), fc.stage
    dyn = Node(H, op(MATMUL, transpose_b=1), [tensor(I8, (3, 9, k), None), tensor(I8, w.shape, w, True, wq)], F32)
    assert dyn.stage == DECLINED, dyn.stage
    bad = Node(H, op(MATMUL, transpose_b=1), [tensor(I8, (2, 9, k), None, False, [(0.02, -3)]),
                                              tensor(I8, w.shape, w, True, wq)], I8, [(0.05, 5)])
    assert bad.stage in (DECLINED, INFER_FAILED), bad.stage  # batch extents 2 and 3 do not broadcast


@pytest.mark.gpu
def test_a_session_gives_its_stream_back(H, orc):
    """Every kernel holds a reference on its session's stream; destroying the session's last kernel destroys it."""
    H.mi355x_provider_session_streams.restype = C.c_int64
    rng = np.random.default_rng(22)
    before = H.mi355x_provider_session_streams()
    a, w, sw, b, ins = _fc_inputs(rng, 4, 16, 32)
    one = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)])
    two = Node(H, op(FC, has_bias=1), _fc_inputs(rng, 4, 16, 32)[4], I8, [(0.05, 5)])
    assert H.mi355x_provider_session_streams() == before + 2  # the harness gives every unlinked node a session of its own
    one.run(a)
    one.close()
    assert H.mi355x_provider_session_streams() == before + 1
    two.close()
    assert H.mi355x_provider_session_streams() == before


@pytest.mark.gpu
def test_a_foreign_device_address_on_an_input_is_not_followed(H, orc):
    """An address on the input tensor that no kernel of this provider published (an application may attach memory of
    another device) is ignored: the kernel reads the host data."""
    rng = np.random.default_rng(15)
    m, n, k = 9, 40, 64
    a, w, sw, b, ins = _fc_inputs(rng, m, n, k)
    node = Node(H, op(FC, has_bias=1), ins, I8, [(0.05, 5)])
    assert node.stage == OK, (node.stage, node.code)
    H.ph_set_input_device_data(node.h, 0x1000)
    got, _ = node.run(a)
    assert np.array_equal(got, orc.matmul_int8(a, w, b, 0.02, -3, sw, np.zeros(n, np.int32), 0.05, 5, 0, True))
    node.close()


@pytest.mark.gpu
def test_dense_3x3_stride_1_is_taken_on_request(H, orc, monkeypatch):
    """Declined by default (x86 builds of the reference run a Winograd kernel there); with MI355X_CONV3X3=exact the
    provider computes the exact convolution, the reference's own choice on ARM64 with dot product."""
    from oracle.pyoracle import conv_shape
    rng = np.random.default_rng(31)
    x = rng.integers(-128, 128, (1, 12, 10, 16), dtype=np.int8)
    w = rng.integers(-128, 128, (24, 3, 3, 16), dtype=np.int8)
    sw = rng.uniform(1e-3, 1e-2, 24).astype(np.float32).astype(np.float64)
    bias = rng.integers(-3000, 3000, 24).astype(np.int32)
    conv = op(CONV, kernel=(3, 3), stride=(1, 1), dilation=(1, 1), pad_mode=1, in_channel=16, out_channel=24, act=1)
    ins = lambda: [tensor(I8, x.shape, None, False, [(0.03, 2)]), tensor(I8, w.shape, w, True, [(s, 0) for s in sw]),
                   tensor(I32, (24,), bias, True)]
    monkeypatch.delenv("MI355X_CONV3X3", raising=False)
    assert Node(H, conv, ins(), I8, [(0.08, -4)]).stage == DECLINED
    monkeypatch.setenv("MI355X_CONV3X3", "exact")
    node = Node(H, conv, ins(), I8, [(0.08, -4)])
    assert node.stage == OK, (node.stage, node.code)
    got, _ = node.run(x)
    shape = conv_shape(1, 12, 10, 16, 24, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1))
    want = orc.conv_int8(x, w, bias, shape, 0.03, 2, sw, np.zeros(24, np.int32), 0.08, -4, 1)
    assert got.shape == want.shape and np.array_equal(got, want)
    node.close()


def test_pinned_allocator_without_a_gpu_still_allocates(H):
    """A session whose device info carries the allocator must keep working where there is no MI355X: the allocator
    initialises the library itself and falls back to ordinary aligned memory."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the page-locked path is covered by the GPU test")
    H.ph_allocator_fallback_selftest.restype = C.c_int32
    assert H.ph_allocator_fallback_selftest() == 0


@pytest.mark.gpu
def test_pinned_allocator_for_the_device_info(H):
    """mindspore_amd/provider/mi355x_allocator.h: DefaultAllocator's contract (reuse of freed blocks within 64x,
    reference counts from 0, -1 for unknown pointers) on page-locked memory that the GPU copies accept."""
    H.ph_allocator_selftest.restype = C.c_int32
    assert H.ph_allocator_selftest() == 0
