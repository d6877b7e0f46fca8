"""Writes the committed golden fixtures from the COMPILED nnacl (oracle/_ref/libnnacl_ref.so), i.e. from the
reference's own C kernels driven through the Lite wrappers' call sequences.  Run in the build container, where the
reference tree is mounted:

    make -C oracle && python tests/golden/make_golden.py [--full]

Outputs (all small):
  small_cases.npz     inputs + expected outputs of small / odd-shaped cases for every entry point
  config_hashes.json  SHA-256 of the inputs and of the reference outputs for the five benchmark configurations at
                      full size (--full also covers the 8192^3 GEMM, about two minutes of CPU time)
"""
import argparse
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from mindspore_amd import workloads as wl  # noqa: E402
from oracle import pyoracle  # noqa: E402
from oracle.pyoracle import conv_shape  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def small_cases(ref):
    rng = np.random.default_rng(20240)
    out = {}
    idx = 0
    # matmul: (m, n, k, peroc, zw_nonzero, bias, act, b_transpose)
    for m, n, k, peroc, zwnz, hb, act, bt in [
        (1, 1, 1, 0, 0, 1, 0, 1), (3, 5, 7, 1, 1, 1, 0, 1), (8, 12, 33, 0, 1, 0, 1, 0), (13, 70, 64, 1, 0, 1, 3, 1),
        (65, 130, 200, 1, 1, 1, 0, 1), (129, 33, 17, 0, 0, 1, 0, 0), (2, 260, 1000, 1, 0, 0, 0, 1),
        (300, 8, 129, 1, 1, 1, 3, 1)]:
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        w_nk = rng.integers(-128, 128, (n, k), dtype=np.int8)
        nf = n if peroc else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = rng.integers(-10, 11, nf).astype(np.int32) if zwnz else np.zeros(nf, np.int32)
        bias = rng.integers(-5000, 5001, n).astype(np.int32) if hb else np.zeros(0, np.int32)
        sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
        so, zo = float(sx * sw.mean() * np.sqrt(k) * 100), int(rng.integers(-20, 21))
        w = w_nk if bt else np.ascontiguousarray(w_nk.T)
        ref.threads = 1 + idx % 4
        c = ref.matmul_int8(a, w, bias if hb else None, sx, zx, sw, zw, so, zo, act, bool(bt))
        p = "mm%d_" % idx
        out.update({p + "a": a, p + "w": w, p + "bias": bias, p + "sw": sw, p + "zw": zw,
                    p + "meta": np.array([sx, zx, so, zo, act, bt, hb], np.float64), p + "c": c})
        idx += 1
    out["mm_count"] = np.array([idx])
    # conv: (b, ih, iw, ic, oc, kernel, stride, dil, pad, peroc, zwnz, bias, act, depthwise)
    idx = 0
    for b, ih, iw, ic, oc, kern, st, dil, pad, peroc, zwnz, hb, act, dw in [
        (1, 9, 9, 3, 8, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), 1, 0, 1, 3, 0),
        (2, 7, 6, 5, 9, (3, 3), (2, 1), (1, 1), (1, 1, 1, 1), 0, 1, 1, 0, 0),
        (1, 8, 8, 16, 20, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), 1, 1, 1, 1, 0),
        (1, 6, 6, 7, 5, (1, 1), (2, 2), (1, 1), (1, 0, 1, 0), 1, 0, 0, 0, 0),
        (1, 10, 10, 4, 6, (5, 3), (1, 1), (2, 1), (4, 4, 1, 1), 0, 0, 1, 3, 0),
        (2, 9, 7, 12, 12, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 1, 1, 1, 3, 1),
        (1, 8, 8, 5, 5, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), 0, 0, 0, 0, 1),
        # 16-channel-aligned images with more than 128 output pixels (the GEMM gathers from the image), the second one
        # a dense 3x3 stride-1 convolution computed as ConvInt8 (what the reference runs on ARM64 with dot product);
        # drawn from a generator of their own so that the cases before and after keep their values
        (1, 24, 24, 16, 12, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2), 1, 1, 1, 3, 0),
        (1, 12, 13, 32, 8, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 1, 0, 1, 1, 0)]:
        shape = conv_shape(b, ih, iw, ic, oc, kern, st, dil, pad)
        main_rng = rng
        if idx >= 7:
            rng = np.random.default_rng(4242 + idx)
        x = rng.integers(-128, 128, (b, ih, iw, ic), dtype=np.int8)
        w = rng.integers(-128, 128, (oc, kern[0], kern[1]) if dw else (oc, kern[0], kern[1], ic), dtype=np.int8)
        nf = oc if peroc else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = rng.integers(-10, 11, nf).astype(np.int32) if zwnz else np.zeros(nf, np.int32)
        bias = rng.integers(-3000, 3001, oc).astype(np.int32) if hb else np.zeros(0, np.int32)
        sx, zx = float(rng.uniform(0.01, 0.05)), int(rng.integers(-20, 21))
        kdim = kern[0] * kern[1] * (1 if dw else ic)
        so, zo = float(sx * sw.mean() * np.sqrt(kdim) * 100), int(rng.integers(-20, 21))
        ref.threads = 1 + idx % 3
        fn = ref.conv_dw_int8 if dw else ref.conv_int8_as_arm64_sdot
        y = fn(x, w, bias if hb else None, shape, sx, zx, sw, zw, so, zo, act)
        p = "cv%d_" % idx
        geom = np.array([kern[0], kern[1], st[0], st[1], dil[0], dil[1], pad[0], pad[1], pad[2], pad[3], dw], np.int32)
        out.update({p + "x": x, p + "w": w, p + "bias": bias, p + "sw": sw, p + "zw": zw, p + "geom": geom,
                    p + "meta": np.array([sx, zx, so, zo, act, hb], np.float64), p + "y": y})
        idx += 1
        rng = main_rng
    out["cv_count"] = np.array([idx])
    # dynamic quant + dynamic matmul
    idx = 0
    for n_el, sym in [(5000, 0), (777, 1), (4096, 0), (1, 0), (100000, 0)]:
        x = (rng.standard_normal(n_el) * rng.uniform(0.1, 10)).astype(np.float32)
        if n_el > 50:
            x[7] = 8.0
        ref.threads = 1 + idx % 4
        q, s, z = ref.dynamic_quant(x, bool(sym))
        p = "dq%d_" % idx
        out.update({p + "x": x, p + "q": q, p + "meta": np.array([s, z, sym], np.float64)})
        idx += 1
    out["dq_count"] = np.array([idx])
    idx = 0
    for m, n, k, peroc, zw0, hb, act, bt in [(5, 9, 17, 1, 0, 1, 0, 1), (33, 70, 64, 0, 3, 0, 1, 1),
                                             (130, 65, 300, 1, 0, 1, 3, 0), (9, 256, 1000, 1, -2, 1, 0, 1)]:
        a = rng.integers(-128, 128, (m, k), dtype=np.int8)
        w_nk = rng.integers(-128, 128, (n, k), dtype=np.int8)
        nf = n if peroc else 1
        sw = rng.uniform(1e-3, 1e-2, nf).astype(np.float32).astype(np.float64)
        zw = np.full(nf, zw0, np.int32)
        bias = rng.standard_normal(n).astype(np.float32) if hb else np.zeros(0, np.float32)
        sx, zx = float(rng.uniform(0.01, 0.1)), int(rng.integers(-128, 128))
        w = w_nk if bt else np.ascontiguousarray(w_nk.T)
        ref.threads = 1 + idx % 3
        c = ref.dynamic_matmul(a, w, bias if hb else None, sx, zx, sw, zw, act, bool(bt))
        p = "dm%d_" % idx
        out.update({p + "a": a, p + "w": w, p + "bias": bias, p + "sw": sw, p + "zw": zw,
                    p + "meta": np.array([sx, zx, act, bt, hb], np.float64), p + "c": c})
        idx += 1
    out["dm_count"] = np.array([idx])
    return out


def config_hashes(ref, full):
    ref.threads = os.cpu_count() or 8
    h = {}
    c1 = wl.fc_c1()
    h["c1"] = dict(inputs=sha(c1["a"]) + sha(c1["w"]), output=sha(ref.matmul_int8(**c1)))
    # c2: per layer, chained
    x, layers = wl.mobilenet_c2()
    cur = x
    h["c2"] = dict(inputs=sha(x))
    for L in layers:
        shape = conv_shape(cur.shape[0], cur.shape[1], cur.shape[2], L["ic"], L["oc"], (L["kernel"],) * 2,
                           (L["stride"],) * 2, (1, 1), L["pad"])
        fn = ref.conv_dw_int8 if L["kind"] == "dw" else ref.conv_int8
        cur = fn(cur, L["w"], L["bias"], shape, L["sx"], L["zx"], L["sw"], L["zw"], L["so"], L["zo"], L["act"])
        h["c2"][L["name"]] = sha(cur)
    # c3
    h["c3"] = {}
    for name, n, k in wl.BERT_SHAPES:
        x = wl.bert_c3_activation(k)
        q, s, z = ref.dynamic_quant(x)
        wt = wl.bert_c3_weights(name, n, k)
        y = ref.dynamic_matmul(q, wt["w"], wt["bias"], s, z, wt["sw"], wt["zw"])
        h["c3"][name] = dict(x=sha(x), q=sha(q), scale=float(s).hex(), zp=int(z), y=sha(y))
    # c4
    h["c4"] = {}
    for name, n, k in wl.DECODE_SHAPES:
        for m in (1, 2, 4, 8):
            g = wl.gemv_c4(name, n, k, m)
            h["c4"]["%s_m%d" % (name, m)] = dict(inputs=sha(g["a"]) + sha(g["w"]), output=sha(ref.matmul_int8(**g)))
    # c5
    h["c5"] = {}
    for size in ([4096, 8192] if full else [4096]):
        g = wl.gemm_c5(size)
        h["c5"][str(size)] = dict(inputs=sha(g["a"]) + sha(g["w"]), output=sha(ref.matmul_int8(**g)))
        print("c5", size, "done in", ref.last_seconds, "s", flush=True)
    return h


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true")
    ap.add_argument("--only-small", action="store_true")
    args = ap.parse_args()
    ref = pyoracle.reference()
    np.savez_compressed(os.path.join(HERE, "small_cases.npz"), **small_cases(ref))
    if args.only_small:
        return
    path = os.path.join(HERE, "config_hashes.json")
    h = config_hashes(ref, args.full)
    if not args.full and os.path.exists(path):
        old = json.load(open(path))
        if "8192" in old.get("c5", {}):
            h["c5"]["8192"] = old["c5"]["8192"]
    json.dump(h, open(path, "w"), indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
