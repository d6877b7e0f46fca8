"""GPU parity on the five benchmark configurations at full size: full-tensor compare against the CPU oracle run in
the same process, and SHA-256 compare against the hashes the compiled nnacl produced in the build container
(tests/golden/config_hashes.json) -- three independent agreements: nnacl (container) <-> oracle (this box) <-> GPU."""
import hashlib
import json
import os

import numpy as np
import pytest

from mindspore_amd import kernels as K
from mindspore_amd import workloads as wl
from mindspore_amd.kernels import QuantParam as QP
from oracle.pyoracle import conv_shape

pytestmark = pytest.mark.gpu

HASHES = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config_hashes.json")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def _qps(sw, zw):
    return [QP(float(s), int(z)) for s, z in zip(np.atleast_1d(sw), np.atleast_1d(zw))]


def _matmul(c):
    return K.MatmulInt8Kernel(c["w"], c["bias"], QP(c["sx"], c["zx"]), _qps(c["sw"], c["zw"]), QP(c["so"], c["zo"]),
                              True, c["act"])


def test_c1_fullconnection(orc):
    c = wl.fc_c1()
    assert sha(c["a"]) + sha(c["w"]) == HASHES["c1"]["inputs"], "synthetic inputs differ from the build container's"
    kern = K.FullconnectionInt8Kernel(c["w"], c["bias"], QP(c["sx"], c["zx"]), _qps(c["sw"], c["zw"]),
                                      QP(c["so"], c["zo"]), c["act"])
    got = kern.run(c["a"])
    assert np.array_equal(got, orc.matmul_int8(**c))
    assert sha(got) == HASHES["c1"]["output"]


def test_c2_mobilenet_block(orc):
    import torch
    orc.set_threads(16)
    x, layers = wl.mobilenet_c2()
    assert sha(x) == HASHES["c2"]["inputs"]
    cur_cpu = x
    cur_gpu = torch.from_numpy(x).cuda()
    for L in layers:
        shape = conv_shape(cur_cpu.shape[0], cur_cpu.shape[1], cur_cpu.shape[2], L["ic"], L["oc"], (L["kernel"],) * 2,
                           (L["stride"],) * 2, (1, 1), L["pad"])
        fn = orc.conv_dw_int8 if L["kind"] == "dw" else orc.conv_int8
        want = fn(cur_cpu, L["w"], L["bias"], shape, L["sx"], L["zx"], L["sw"], L["zw"], L["so"], L["zo"], L["act"])
        kern = K.ConvolutionInt8Kernel(L["w"], L["bias"], QP(L["sx"], L["zx"]), _qps(L["sw"], L["zw"]),
                                       QP(L["so"], L["zo"]), (L["stride"],) * 2, (1, 1), L["pad"],
                                       L["oc"] if L["kind"] == "dw" else 1, L["act"])
        # per layer from the oracle's input (host tensors) and end-to-end chained on the device
        assert np.array_equal(kern.run(cur_cpu), want), L["name"]
        cur_gpu = kern.run(cur_gpu)
        torch.cuda.synchronize()
        assert np.array_equal(cur_gpu.cpu().numpy(), want), L["name"] + " (chained)"
        assert sha(want) == HASHES["c2"][L["name"]], L["name"]
        cur_cpu = want


@pytest.mark.parametrize("name,n,k", wl.BERT_SHAPES)
def test_c3_bert_dynamic(orc, name, n, k):
    import torch
    orc.set_threads(16)
    x = wl.bert_c3_activation(k)
    wt = wl.bert_c3_weights(name, n, k)
    g = HASHES["c3"][name]
    assert sha(x) == g["x"]
    dq = K.DynamicQuantKernel(False)
    mm = K.MatmulDynamicInt8Kernel(wt["w"], wt["bias"], _qps(wt["sw"], wt["zw"]))
    xt = torch.from_numpy(x).cuda()
    q, qp = dq.run(xt)
    q_ref, s_ref, z_ref = orc.dynamic_quant(x)
    # north-star tolerance: scale within 1 ulp of fp32; measured: exact
    assert qp.scale == s_ref and qp.zero_point == z_ref
    assert float(s_ref).hex() == g["scale"] and z_ref == g["zp"]
    assert np.array_equal(q.cpu().numpy(), q_ref) and sha(q_ref) == g["q"]
    y = mm.run(q, params_dev=dq.device_params())
    torch.cuda.synchronize()
    want = orc.dynamic_matmul(q_ref, wt["w"], wt["bias"], s_ref, z_ref, wt["sw"], wt["zw"])
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert sha(want) == g["y"]


@pytest.mark.parametrize("name,n,k", wl.DECODE_SHAPES)
def test_c4_decode_gemv(orc, name, n, k):
    orc.set_threads(16)
    kern = None
    for m in (1, 2, 4, 8):
        c = wl.gemv_c4(name, n, k, m)
        g = HASHES["c4"]["%s_m%d" % (name, m)]
        assert sha(c["a"]) + sha(c["w"]) == g["inputs"]
        kern = _matmul(c)
        got = kern.run(c["a"])
        assert np.array_equal(got, orc.matmul_int8(**c)), (name, m)
        assert sha(got) == g["output"]
        kern.close()
    # rows 3, 5, 6, 7 (no golden hash; oracle only)
    c = wl.gemv_c4(name, n, k, 8)
    kern = _matmul(c)
    for m in (3, 5, 6, 7):
        sub = dict(c)
        sub["a"] = np.ascontiguousarray(c["a"][:m])
        assert np.array_equal(kern.run(sub["a"]), orc.matmul_int8(**sub)), (name, m)


@pytest.mark.parametrize("size", [4096, 8192])
def test_c5_square_gemm(orc, size):
    orc.set_threads(16)
    c = wl.gemm_c5(size)
    g = HASHES["c5"][str(size)]
    assert sha(c["a"]) + sha(c["w"]) == g["inputs"]
    got = _matmul(c).run(c["a"])
    assert sha(got) == g["output"]
    if size == 4096:
        assert np.array_equal(got, orc.matmul_int8(**c))
    else:
        # full-size oracle run would take a while: the GEMM is row-independent, so check a spread of rows
        rows = np.unique(np.concatenate([np.arange(0, 300), np.arange(size - 300, size),
                                         np.random.default_rng(1).integers(0, size, 424)]))
        sub = dict(c)
        sub["a"] = np.ascontiguousarray(c["a"][rows])
        assert np.array_equal(got[rows], orc.matmul_int8(**sub))
