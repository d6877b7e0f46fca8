#!/usr/bin/env python3
"""Benchmark of the MI355X int8 hot path.

One "step" = one pass of the hot path over one batch of synthetic input.  The headline workload is the 4096^3
int8 GEMM of benchmark configuration 5 (int8 x int8 -> int32 on the matrix cores with the fused per-channel
requantising epilogue); the decode GEMV (configuration 4, batch 1), DynamicQuant and the BERT dynamic MatMuls
(configuration 3) are timed in the same run and reported under "extra".  Inputs are resident in HBM before the
timed region.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload gemm4096|gemm8192] [--no-cpu] [--no-extra]
                    [--calibrate] [--conv3x3] [--dynquant] [--bert] [--c2]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0  # MI355X dense int8 MFMA peak, TOP/s (5.0 POP/s)
PEAK_HBM_GBPS = 8000.0   # MI355X HBM3E peak, GB/s

HEADLINE_KERNEL = "mi::gemm_kblock_kernel<0, false, true>"
# HBM-side bytes per launch of the dominant kernel come from `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of
# this script, each scaled by what the same counter reads for the 256 MiB copy of --calibrate.  The figures are read
# from the committed summary of those runs, which also names the kernel and the commit it was measured at, so that
# a number that no longer belongs to the current kernel shows.
TRAFFIC_SUMMARY = {"gemm4096": os.path.join(ROOT, "profiles", "gemm_kblock_kernel_gemm4096.txt"), "gemm8192": None}


def measured_traffic(workload):
    """{bytes, kernel, commit} from the `key: value` lines of the profile summary, or None."""
    path = TRAFFIC_SUMMARY.get(workload)
    if not path or not os.path.exists(path):
        return None
    kv = {}
    for line in open(path):
        key, sep, val = line.partition(":")
        if sep and key.strip() in ("traffic_bytes_per_launch", "kernel", "measured_at_commit"):
            kv[key.strip()] = val.strip()
    if "traffic_bytes_per_launch" not in kv:
        return None
    return dict(bytes=int(kv["traffic_bytes_per_launch"]), kernel=kv.get("kernel"), commit=kv.get("measured_at_commit"))


def roofline_fields(ops, nbytes, ms):
    """Where a launch of `ops` integer operations and `nbytes` algorithmic bytes that took `ms` stands against both
    roofs; `bound` names the roof whose floor (ops / MFMA peak, bytes / HBM peak) is the higher one for this shape and
    `frac` is the fraction of that roof."""
    secs = ms * 1e-3
    f_mfma = ops / secs / 1e12 / PEAK_INT8_TOPS if ops else 0.0
    f_hbm = nbytes / secs / 1e9 / PEAK_HBM_GBPS
    bound = "mfma" if ops / (PEAK_INT8_TOPS * 1e12) > nbytes / (PEAK_HBM_GBPS * 1e9) else "hbm"
    return dict(bound=bound, frac=f_mfma if bound == "mfma" else f_hbm, ops=ops, algorithmic_bytes=int(nbytes),
                frac_of_int8_peak=f_mfma, frac_of_hbm_peak=f_hbm)


def host_cores():
    """Threads the CPU baseline runs on: every core this process may use; a thread-count limit the environment sets
    (OMP_NUM_THREADS, the box's CPU share) is respected.  Returns (threads used, what nproc reports)."""
    nproc = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    used = nproc
    limit = os.environ.get("OMP_NUM_THREADS", "")
    if limit.isdigit() and int(limit) > 0:
        used = min(used, int(limit))
    return used, nproc


def time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return start.elapsed_time(stop) / steps, wall * 1e3 / steps  # ms per step by HIP events, by host clock


def time_in_graph(fn, steps, warmup, calls=10, settle_ms=40.0):
    """ms per call of fn with `calls` invocations captured in one HIP graph and the graph replayed: what the GPU
    needs per call once the Python host's per-call cost (about 10 us here) is out of the way, as it is for a C++
    caller of the C ABI."""
    import torch
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fn()  # workspaces and one-time copies are made outside the capture
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(calls):
                fn()
    torch.cuda.synchronize()
    # replayed for about 40 ms first: the timed replays start from the state the power management settles in under
    # this load (see settle), not from the transient after an idle device
    t0 = time.perf_counter()
    for _ in range(200):
        for _ in range(25):
            graph.replay()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 > settle_ms * 1e-3:
            break
    ms, _ = time_steps(graph.replay, max(20, steps // calls), warmup)  # at least 200 calls: a few ms
    return ms / calls


def make_matmul(c):
    from mindspore_amd import kernels as K
    qp = [K.QuantParam(float(s), int(z)) for s, z in zip(c["sw"], c["zw"])]
    return K.MatmulInt8Kernel(c["w"], c["bias"], K.QuantParam(c["sx"], c["zx"]), qp, K.QuantParam(c["so"], c["zo"]),
                              True, c["act"])


def settle(kern, a, out, min_ms=60.0, chunk=50):
    """Launches the GEMM back to back from an idle device until at least `min_ms` of it have run, timing every chunk
    of launches.  Under this load the power management first over-corrects -- launches 10 to ~150 after idle run
    10-20 % slower than the first ones -- and settles after about 20 ms at a rate it then holds; a region of a few
    dozen launches right after idle measures that transient, not the kernel.  The timed steps therefore start from
    the settled state, and the series is reported so that the transient is visible."""
    import torch
    series, total, launches = [], 0.0, 0
    while total < min_ms and len(series) < 64:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(chunk):
            kern.run(a, out=out)
        stop.record()
        torch.cuda.synchronize()  # (a wait of microseconds: the device does not leave the state it is in)
        ms = start.elapsed_time(stop)
        series.append(round(ms * 1e3 / chunk, 2))
        total += ms
        launches += chunk
    return dict(launches=launches, ms=total, launches_per_chunk=chunk, us_per_launch_by_chunk=series,
                note="untimed launches from an idle device before the warm-up and the timed steps: the shader clock "
                     "needs about 20 ms under this load to settle")


def sustained_probe():
    """Buffers of bench_sustained, made before the device is brought to its settled state: a host pause of a few
    milliseconds between two timed regions is enough for the power management to start over."""
    import numpy as np
    import torch
    from mindspore_amd import lib
    D = lib.load_diag()
    ops_t = torch.from_numpy(np.random.default_rng(0).integers(-128, 128, 32768, dtype=np.int8)).cuda()
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()
    return D, ops_t, clocks


def bench_sustained(kern, a, out, size, probe, launches=400):
    """The same GEMM launched back to back for at least 20 ms, straight after the timed steps, i.e. from the settled
    state (see settle).  The shader clock is read by a 0.3 ms matrix-pipe loop (in-kernel cycle counter against the
    100 MHz counter) queued right behind the last launch, on operands drawn like the GEMM's."""
    import torch
    from mindspore_amd import lib
    D, ops_t, clocks = probe
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(launches):
        kern.run(a, out=out)
    stop.record()
    lib.check(D.mi_diag_mfma_rate(ops_t.data_ptr(), 1024, 256, clocks.data_ptr(), _stream()), "mi_diag_mfma_rate")
    torch.cuda.synchronize()
    total_ms = start.elapsed_time(stop)
    ms = total_ms / launches
    c = clocks.cpu().numpy()
    tops = 2.0 * size ** 3 / (ms * 1e-3) / 1e12
    return dict(launches=launches, total_ms=total_ms, ms_per_launch=ms, tops=tops, frac_of_int8_peak=tops / PEAK_INT8_TOPS,
                shader_clock_ghz_right_after=float(c[0]) / (float(c[1]) * 10.0))


def bench_gemm(size, steps, warmup, host_path=False, sustained=False):
    import torch
    from mindspore_amd import workloads as wl
    c = wl.gemm_c5(size)
    make_matmul(c).close()  # the first create of a process also loads the code object
    t0 = time.perf_counter()
    kern = make_matmul(c)
    torch.cuda.synchronize()
    prepare_ms = (time.perf_counter() - t0) * 1e3  # Prepare(): quant parameters, weight sums, packing, upload
    a = torch.from_numpy(c["a"]).cuda()
    out = torch.empty((size, size), dtype=torch.int8, device="cuda")
    probe = sustained_probe() if sustained else None
    ops = 2.0 * size * size * size
    # first the region exactly as asked for, straight from the idle device (0.2 s without GPU work precede it): this
    # is the power management's transient (see settle), reported beside the settled figure
    torch.cuda.synchronize()
    time.sleep(0.2)
    idle_ms, _ = time_steps(lambda: kern.run(a, out=out), steps, warmup)
    from_idle = dict(ms_per_step=idle_ms, tops=ops / (idle_ms * 1e-3) / 1e12,
                     frac_of_int8_peak=ops / (idle_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, steps=steps, warmup=warmup,
                     note="the same timed region started from an idle device, before the untimed settling launches")
    settled = settle(kern, a, out, chunk=50 if size <= 4096 else 10)
    ev_ms, host_ms = time_steps(lambda: kern.run(a, out=out), steps, warmup)
    res = dict(ms=ev_ms, host_ms=host_ms, tops=ops / (ev_ms * 1e-3) / 1e12, ops=ops, case=c, prepare_ms=prepare_ms,
               settled=settled, from_idle=from_idle)
    if sustained:
        res["sustained"] = bench_sustained(kern, a, out, size, probe)
    if host_path:
        # the boundary as the provider uses it today: host tensors in and out (pinned staging + PCIe both ways)
        kern.run(c["a"])
        t0 = time.perf_counter()
        for _ in range(3):
            kern.run(c["a"])
        res["host_path_ms"] = (time.perf_counter() - t0) / 3 * 1e3
    return res


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def bench_tile_fixed_cost(size=8192, ks=(1024, 4096, 8192), steps=20):
    """What a 256 x 256 tile costs beyond its K loop when a CU runs several tiles one after the other (1024 tiles on
    256 CUs at 8192 x 8192): the launch time at three K, a line through them, and its intercept divided by the tiles
    per CU.  That intercept is dispatch + parameter fetch + first operand fetch + epilogue of one tile; a persistent
    kernel that prefetches the next tile under the epilogue can at most save the part of it that is not epilogue."""
    import numpy as np
    import torch
    from mindspore_amd import kernels as K
    rng = np.random.default_rng(5)
    a_full = torch.from_numpy(rng.integers(-128, 128, (size, max(ks)), dtype=np.int8)).cuda()
    out = torch.empty((size, size), dtype=torch.int8, device="cuda")
    sw = rng.uniform(1e-4, 1e-2, size).astype(np.float32)
    times = {}
    for k in ks:
        w = rng.integers(-128, 128, (size, k), dtype=np.int8)
        so = float(np.float32(0.02 * float(np.mean(sw)) * np.sqrt(k) * 150.0))
        kern = K.MatmulInt8Kernel(w, None, K.QuantParam(0.02, 7), [K.QuantParam(float(s), 0) for s in sw],
                                  K.QuantParam(so, 0), True, 0, decode_pack=False)
        a = a_full[:, :k].contiguous()
        for _ in range(60):  # ~20 ms: the settled state
            kern.run(a, out=out)
        ms, _ = time_steps(lambda: kern.run(a, out=out), steps, 2)
        times[k] = ms * 1e3
        kern.close()
    xs, ys = np.array(sorted(times)), np.array([times[k] for k in sorted(times)])
    slope, intercept = np.polyfit(xs, ys, 1)
    tiles_per_cu = (size // 256) ** 2 / 256.0
    return dict(us_by_k={int(k): float(v) for k, v in times.items()}, us_per_128_bytes_of_k=float(slope * 128),
                fixed_us_per_launch=float(intercept), tiles_per_cu=tiles_per_cu,
                fixed_us_per_tile=float(intercept / tiles_per_cu),
                note="launch time = fixed + K x slope; fixed / tiles per CU is what one tile costs outside its K loop "
                     "(of which the epilogue is 5.3-5.7 us)")


def bench_hbm_read(steps, warmup):
    """What a kernel that only reads can reach on this device: the library's plain read stream over 48 MiB slices
    (the size of one decode weight matrix) of a 3 GiB buffer, so no slice is still in the 256 MB Infinity Cache when
    it is read again."""
    import torch
    from mindspore_amd import lib
    L = lib.load_diag()
    slice_bytes, n_slices = 48 << 20, 64
    buf = torch.ones(slice_bytes * n_slices, dtype=torch.int8, device="cuda")
    state = {"i": 0}
    def step():
        i = state["i"] = (state["i"] + 1) % n_slices
        lib.check(L.mi_diag_stream_read(buf.data_ptr() + i * slice_bytes, slice_bytes, _stream()), "mi_diag_stream_read")
    ms, _ = time_steps(step, max(steps, 40), warmup)
    del buf
    return dict(bytes=slice_bytes, ms=ms, gbps=slice_bytes / (ms * 1e-3) / 1e9)


def bench_mfma_rate():
    """The matrix pipe alone (register operands, no LDS, no memory) on all-zero operands and on operands drawn like
    the GEMM's (uniform int8): the sustained shader clock, hence the rate, depends on the operand data."""
    import numpy as np
    import torch
    from mindspore_amd import lib
    L = lib.load_diag()
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    out = {}
    iters, wgs = 40000, 256
    for name, data in (("zero_operands", np.zeros(32768, np.int8)),
                       ("uniform_int8_operands", np.random.default_rng(0).integers(-128, 128, 32768, dtype=np.int8))):
        ops = torch.from_numpy(data).cuda()
        fn = lambda: lib.check(L.mi_diag_mfma_rate(ops.data_ptr(), iters, wgs, clocks.data_ptr(), _stream()),
                               "mi_diag_mfma_rate")
        ms, _ = time_steps(fn, 3, 1)
        c = clocks.cpu().numpy()
        out[name] = dict(tops=wgs * 4 * iters * 16 * 65536.0 / (ms * 1e-3) / 1e12, ms=ms,
                         shader_clock_ghz=float(c[0]) / (float(c[1]) * 10.0))
    return out


def bench_vendor_int_mm(size, steps):
    """Yardstick only (not part of the product path): the vendor GEMM library behind torch._int_mm on the same
    operand distribution -- int8 x int8 -> int32, no requantisation, 16.8 MB less output compression work than the
    kernel under test.  Shows what a tuned library reaches on this box under the same data-dependent clock."""
    import torch
    try:
        a = torch.randint(-128, 128, (size, size), dtype=torch.int8, device="cuda")
        b = torch.randint(-128, 128, (size, size), dtype=torch.int8, device="cuda")
        ms, _ = time_steps(lambda: torch._int_mm(a, b), steps, 3)
    except Exception as ex:  # noqa: BLE001 -- an optional yardstick must never fail the benchmark
        return dict(error=str(ex)[:200])
    return dict(ms=ms, tops=2.0 * size ** 3 / (ms * 1e-3) / 1e12, what="torch._int_mm, int32 output, uniform int8")


def native_bench(*args, env=None):
    """Runs mindspore_amd/native_bench (C++ host over the C ABI) as a child process and returns its JSON, or None when
    the binary is not built."""
    import subprocess
    exe = os.path.join(ROOT, "mindspore_amd", "native_bench")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=300, check=True,
                             env=dict(os.environ, **(env or {})))
        return json.loads(out.stdout.strip().splitlines()[-1])
    except Exception as ex:  # noqa: BLE001
        return dict(error=str(ex)[:200])


def bench_gemv(steps, warmup, m=1):
    """Decode step: the five 7B-class layer matrices, three layers' worth of distinct weights (606 MB) cycled so the
    256 MB Infinity Cache cannot hold the working set.  Outputs are preallocated; one step = 15 launches."""
    import torch
    from mindspore_amd import workloads as wl
    kerns, acts, outs, total_bytes = [], [], [], 0
    for layer in range(3):
        for name, n, k in wl.DECODE_SHAPES:
            c = wl.gemv_c4(name, n, k, m, seed=layer)
            kerns.append(make_matmul(c))
            acts.append(torch.from_numpy(c["a"]).cuda())
            outs.append(torch.empty((m, n), dtype=torch.int8, device="cuda"))
            total_bytes += n * k + m * k + m * n + 16 * n
    def step():
        for kern, a, o in zip(kerns, acts, outs):
            kern.run(a, out=o)
    ev_ms, _ = time_steps(step, steps, warmup)
    gbps = total_bytes / (ev_ms * 1e-3) / 1e9
    return dict(m=m, launches_per_step=len(kerns), ms_per_step=ev_ms, us_per_launch=ev_ms * 1e3 / len(kerns),
                bytes_per_step=total_bytes, gbps=gbps, frac_of_hbm_peak=gbps / PEAK_HBM_GBPS)


def bench_bert(steps, warmup):
    import torch
    from mindspore_amd import kernels as K
    from mindspore_amd import workloads as wl
    out = {}
    x = torch.from_numpy(wl.bert_c3_activation(768)).cuda()
    dq = K.DynamicQuantKernel(False)
    ms = time_in_graph(lambda: dq.run(x, fetch_params=False), steps, warmup)
    nbytes = x.numel() * 5
    out["dynquant_4096x768"] = dict(ms=ms, gbps=nbytes / (ms * 1e-3) / 1e9, **roofline_fields(0, nbytes, ms))
    # the same two kernels on a tensor large enough to leave the launch-latency regime (16x the BERT activation)
    xl = torch.randn((65536, 768), device="cuda", dtype=torch.float32)
    ms, _ = time_steps(lambda: dq.run(xl, fetch_params=False), steps, warmup)
    nbytes = xl.numel() * 5
    out["dynquant_65536x768"] = dict(ms=ms, gbps=nbytes / (ms * 1e-3) / 1e9, **roofline_fields(0, nbytes, ms),
                                     note="algorithmic bytes (4 read + 1 written per element); the second pass re-reads "
                                          "201 MB, of which the Infinity Cache holds only part")
    del xl
    q, _ = dq.run(x, fetch_params=False)
    total_ops, total_ms = 0.0, 0.0
    for name, n, k in wl.BERT_SHAPES:
        wt = wl.bert_c3_weights(name, n, k)
        mm = K.MatmulDynamicInt8Kernel(wt["w"], wt["bias"], [K.QuantParam(float(s), 0) for s in wt["sw"]])
        qa = q if k == 768 else torch.randint(-128, 127, (4096, k), dtype=torch.int8, device="cuda")
        ms = time_in_graph(lambda: mm.run(qa, params_dev=dq.device_params()), steps, warmup)
        ops = 2.0 * 4096 * n * k
        nbytes = 4096 * k + n * k + 4 * 4096 * n + 12 * n  # int8 activations and weights, fp32 output, per-channel scale / sum / bias
        # what a kernel that only writes the same fp32 output takes (a fill of the output tensor, timed the same way):
        # the part of the launch that no arrangement of the GEMM can take away
        y = torch.empty((4096, n), dtype=torch.float32, device="cuda")
        fill_ms = time_in_graph(lambda: y.fill_(1.0), steps, warmup)
        del y
        out["dynmm_" + name] = dict(ms=ms, tops=ops / (ms * 1e-3) / 1e12, gbps=nbytes / (ms * 1e-3) / 1e9,
                                    output_fill_only_us=fill_ms * 1e3, **roofline_fields(ops, nbytes, ms))
        total_ops += ops
        total_ms += ms
    out["dynmm_total_tops"] = total_ops / (total_ms * 1e-3) / 1e12
    out["dynmm_total_us"] = total_ms * 1e3
    return out


def bench_small_configs(steps, warmup):
    """Configuration 1 (FullConnection 128x768x768) and configuration 2 (MobileNetV2-style block, device-resident
    chain of stem 3x3 s2, 1x1 expand, 3x3 depthwise, 1x1 project): latency per layer, algorithmic bytes moved."""
    import numpy as np
    import torch
    from mindspore_amd import kernels as K
    from mindspore_amd import workloads as wl
    out = {}
    c = wl.fc_c1()
    fc = make_matmul(c)
    a = torch.from_numpy(c["a"]).cuda()
    o = torch.empty((128, 768), dtype=torch.int8, device="cuda")
    ms = time_in_graph(lambda: fc.run(a, out=o), steps, warmup)
    out["c1_fc_128x768x768"] = dict(us=ms * 1e3, tops=2.0 * 128 * 768 * 768 / (ms * 1e-3) / 1e12,
                                    **roofline_fields(2.0 * 128 * 768 * 768, 128 * 768 + 768 * 768 + 128 * 768 + 16 * 768, ms))
    x, layers = wl.mobilenet_c2()
    cur = torch.from_numpy(x).cuda()
    kerns, ins = [], []
    for L in layers:
        qp = [K.QuantParam(float(sc), int(z)) for sc, z in zip(L["sw"], L["zw"])]
        kern = K.ConvolutionInt8Kernel(L["w"], L["bias"], K.QuantParam(L["sx"], L["zx"]), qp,
                                       K.QuantParam(L["so"], L["zo"]), (L["stride"],) * 2, (1, 1), L["pad"],
                                       L["oc"] if L["kind"] == "dw" else 1, L["act"])
        kerns.append(kern)
        ins.append(cur)
        cur = kern.run(cur)
    outs = [kern.run(xin) for kern, xin in zip(kerns, ins)]
    block_bytes, block_ops = 0, 0.0
    for L, kern, xin, yout in zip(layers, kerns, ins, outs):
        ms = time_in_graph(lambda: kern.run(xin, out=yout), steps, warmup)
        nbytes = xin.numel() + yout.numel() + L["w"].size + 16 * L["oc"]
        kdim = L["kernel"] ** 2 * (1 if L["kind"] == "dw" else L["ic"])
        out["c2_" + L["name"]] = dict(us=ms * 1e3, in_shape=list(xin.shape), out_shape=list(yout.shape),
                                      gbps=nbytes / (ms * 1e-3) / 1e9, **roofline_fields(2.0 * yout.numel() * kdim, nbytes, ms))
        block_bytes += nbytes
        block_ops += 2.0 * yout.numel() * kdim
    # the whole block as one captured HIP graph (five kernels), replayed: what the GPU needs once the host's
    # per-call cost is out of the way
    def chain():
        cur = ins[0]
        for kern, yout in zip(kerns, outs):
            cur = kern.run(cur, out=yout)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        chain()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            chain()
    torch.cuda.synchronize()
    ms, _ = time_steps(graph.replay, steps, warmup)
    total_us = ms * 1e3
    out["c2_block_graph_us"] = total_us
    out["c2_block"] = dict(us=total_us, kernels=len(kerns), gbps=block_bytes / (total_us * 1e-6) / 1e9,
                           note="stem, expand, depthwise and project replayed as one HIP graph; algorithmic bytes are "
                                "the sum over the four layers (every intermediate tensor written once and read once)",
                           **roofline_fields(block_ops, block_bytes, ms))
    # a mid-network 3x3 convolution: the GEMM gathers its activation operand from the image
    kern, xin, yout, nbytes = make_conv3x3()
    us = time_in_graph(lambda: kern.run(xin, out=yout), steps, 3) * 1e3
    out["conv3x3_b32_56x56x64"] = dict(us=us, tops=2.0 * yout.numel() * 9 * 64 / (us * 1e-6) / 1e12,
                                       **roofline_fields(2.0 * yout.numel() * 9 * 64, nbytes, us * 1e-3))
    return out


def make_conv3x3():
    """Batch 32, 56 x 56 x 64 -> 64 channels, 3x3, stride 1, pad 1 (taken with MI_CONV_3X3_EXACT)."""
    import numpy as np
    import torch
    from mindspore_amd import kernels as K
    rng = np.random.default_rng(3)
    xin = torch.from_numpy(rng.integers(-128, 128, (32, 56, 56, 64), dtype=np.int8)).cuda()
    wt = rng.integers(-128, 128, (64, 3, 3, 64), dtype=np.int8)
    qp = [K.QuantParam(float(sc), 0) for sc in rng.uniform(1e-3, 1e-2, 64)]
    kern = K.ConvolutionInt8Kernel(wt, None, K.QuantParam(0.02, 3), qp, K.QuantParam(0.5, -2), (1, 1), (1, 1),
                                   (1, 1, 1, 1), 1, 0, exact_3x3=True)
    yout = kern.run(xin)
    return kern, xin, yout, int(xin.numel() + yout.numel() + wt.size)


def cpu_baseline(case, size):
    """nnacl's CPU path (compiled from the reference tree, oracle/_ref) -- or the restatement if that library did
    not travel -- on a bounded sample: the first `rows` activation rows of the same GEMM on all host cores (about 20
    core-seconds), and the first 64 rows on one thread."""
    from oracle import pyoracle
    cores, nproc = host_cores()
    if pyoracle.Reference.available():
        eng, kind = pyoracle.reference(), "reference"
    else:
        eng, kind = pyoracle.oracle(), "port"

    def run(rows, threads):
        sub = dict(case)
        sub["a"] = case["a"][:rows].copy()
        if kind == "reference":
            eng.threads = threads
            eng.matmul_int8(**sub)
            secs = eng.last_seconds
        else:
            eng.set_threads(threads)
            t0 = time.perf_counter()
            eng.matmul_int8(**sub)
            secs = time.perf_counter() - t0
        return 2.0 * rows * size * size / secs / 1e12, secs

    rows = 1024 if size <= 4096 else 256
    runs = sorted(run(rows, cores) for _ in range(3))  # median of three
    tops, secs = runs[1]
    tops1, secs1 = run(64 if size <= 4096 else 16, 1)
    return dict(value=tops, unit="TOP/s", cores=cores, nproc=nproc, kind=kind, seconds=secs,
                runs_tops=[r[0] for r in runs], statistic="median of 3 runs",
                sample="first %d of %d activation rows of the same %d^3 GEMM (A-pack + row sums + MatmulInt8Opt "
                       "column stripes on %d threads)" % (rows, size, size, cores),
                single_thread=dict(value=tops1, unit="TOP/s", cores=1, seconds=secs1,
                                   sample="first %d rows" % (64 if size <= 4096 else 16)))


def cpu_side_by_side():
    """The reference's CPU path on the other configurations (same engine and thread count as cpu_baseline), a few
    seconds in total: decode GEMV (QKV matrix, one row), DynamicQuant 4096x768, the BERT QKV dynamic MatMul on its
    first 256 rows, configuration 1, and the four layers of configuration 2."""
    from oracle import pyoracle
    from mindspore_amd import workloads as wl
    cores, _ = host_cores()
    if pyoracle.Reference.available():
        eng, kind = pyoracle.reference(), "reference"
        eng.threads = cores
    else:
        eng, kind = pyoracle.oracle(), "port"
        eng.set_threads(cores)

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return eng.last_seconds if kind == "reference" else time.perf_counter() - t0

    out = {"kind": kind, "cores": cores}
    name, n, k = wl.DECODE_SHAPES[0]
    c = wl.gemv_c4(name, n, k, 1, seed=0)
    secs = timed(lambda: eng.matmul_int8(**{kk: c[kk] for kk in ("a", "w", "bias", "sx", "zx", "sw", "zw", "so", "zo", "act")}))
    out["gemv_%s_m1" % name] = dict(ms=secs * 1e3, gbps=(n * k + k + n + 16 * n) / secs / 1e9)
    x = wl.bert_c3_activation(768)
    secs = timed(lambda: eng.dynamic_quant(x))
    out["dynquant_4096x768"] = dict(ms=secs * 1e3, gbps=x.size * 5 / secs / 1e9)
    q, sx, zx = eng.dynamic_quant(x)
    bname, bn, bk = wl.BERT_SHAPES[0]
    wt = wl.bert_c3_weights(bname, bn, bk)
    rows = 256
    secs = timed(lambda: eng.dynamic_matmul(q[:rows], wt["w"], wt["bias"], sx, zx, wt["sw"], np_zeros(bn)))
    out["dynmm_%s_first_%d_rows" % (bname, rows)] = dict(ms=secs * 1e3, tops=2.0 * rows * bn * bk / secs / 1e12)
    c1 = wl.fc_c1()
    secs = timed(lambda: eng.matmul_int8(**{kk: c1[kk] for kk in ("a", "w", "bias", "sx", "zx", "sw", "zw", "so", "zo", "act")}))
    out["c1_fc_128x768x768"] = dict(us=secs * 1e6)
    xin, layers = wl.mobilenet_c2()
    cur, total = xin, 0.0
    for L in layers:
        shape = pyoracle.conv_shape(cur.shape[0], cur.shape[1], cur.shape[2], L["ic"], L["oc"], (L["kernel"],) * 2,
                                    (L["stride"],) * 2, (1, 1), L["pad"])
        fn = eng.conv_dw_int8 if L["kind"] == "dw" else eng.conv_int8
        res = {}
        secs = timed(lambda: res.setdefault("y", fn(cur, L["w"], L["bias"], shape, L["sx"], L["zx"], L["sw"], L["zw"],
                                                    L["so"], L["zo"], L["act"])))
        out["c2_" + L["name"]] = dict(us=secs * 1e6)
        total += secs
        cur = res["y"]
    out["c2_block_us"] = total * 1e6
    return out


def np_zeros(n):
    import numpy as np
    return np.zeros(n, np.int32)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="gemm4096", choices=["gemm4096", "gemm8192"])
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch the library's 256 MiB device copy three times (known traffic, for scaling "
                         "the profiler's FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--conv3x3", action="store_true",
                    help="also launch the batch-32 3x3 convolution of the extras 20 times (for profiling that kernel)")
    ap.add_argument("--bert", action="store_true",
                    help="also launch each of the four BERT dynamic MatMuls of configuration 3 twenty times (for "
                         "profiling their kernels; mindspore_amd/native_bench bert does the same without Python)")
    ap.add_argument("--c2", action="store_true",
                    help="also run the four layers of configuration 2 twenty times each (for profiling their kernels)")
    ap.add_argument("--dynquant", action="store_true",
                    help="also run DynamicQuant on the 4096 x 768 activation of configuration 3 a hundred times (for "
                         "profiling its two kernels)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this hot path is a single-GPU path; only --gpus 1 is supported (got %d)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from mindspore_amd import lib
    lib.init(0)  # raises if the HIP library is missing or the GPU is not gfx950

    size = 4096 if args.workload == "gemm4096" else 8192
    g = bench_gemm(size, args.steps, args.warmup, host_path=not args.no_extra, sustained=not args.no_extra)
    extra = {}
    if "sustained" in g:
        extra["gemm%d_sustained" % size] = g["sustained"]

    def section(name, fn):
        """An extra must never cost the headline line: a failure is recorded under its name."""
        try:
            return fn()
        except Exception as ex:  # noqa: BLE001
            extra[name + "_error"] = "%s: %s" % (type(ex).__name__, str(ex)[:300])
            return None

    if not args.no_extra:
        other = 8192 if size == 4096 else 4096
        o = section("gemm%d" % other, lambda: bench_gemm(other, max(3, args.steps // 5), 2))
        if o:
            extra["gemm%d" % other] = dict(ms=o["ms"], tops=o["tops"], frac_of_int8_peak=o["tops"] / PEAK_INT8_TOPS)
        if size == 4096:
            fx = section("gemm8192_fixed_cost_per_tile", bench_tile_fixed_cost)
            if fx:
                extra["gemm8192_fixed_cost_per_tile"] = fx
        mf = section("mfma_only", bench_mfma_rate)
        if mf:
            extra["mfma_only"] = mf
            extra["gemm%d_frac_of_mfma_only_same_data" % size] = g["tops"] / mf["uniform_int8_operands"]["tops"]
        extra["vendor_library_gemm%d" % size] = bench_vendor_int_mm(size, max(10, args.steps // 2))
        rd = section("hbm_read_stream", lambda: bench_hbm_read(args.steps, 3))
        if rd:
            extra["hbm_read_stream"] = rd
        # the decode numbers come from the native host: a Python caller needs about as long per call as one of these
        # kernels runs; the Python-driven figures are kept beside them
        nread = native_bench("read", 48, 64, 4)
        if nread and "gbps" in nread:
            extra["hbm_read_stream_native_host"] = nread
        for m in (1, 2, 4, 8, 32):
            nat = native_bench("decode", m, 3, 1000, 100)  # ~0.1 s of launches after ~10 ms of warm-up: the settled rate
            py = section("gemv_decode_m%d_python_host" % m, lambda: bench_gemv(max(5, args.steps // 2), 3, m)) \
                if m in (1, 8) else None
            if nat and "gbps" in nat:
                best = dict(nat, host="native C++ over the C ABI")
            elif py:
                best = dict(py, host="python/ctypes")
            else:
                continue
            best["frac_of_hbm_peak"] = best["gbps"] / PEAK_HBM_GBPS
            if py:
                best["python_host"] = dict(ms_per_step=py["ms_per_step"], gbps=py["gbps"])
            if "host" in best and best["host"].startswith("native"):
                best["note"] = "gate and up, which share their input, go out as one launch (mi_matmul_run_group)"
                solo = native_bench("decode", m, 3, 1000, 100, env={"NATIVE_BENCH_NO_GROUP": "1"})
                if solo and "gbps" in solo:
                    best["one_launch_per_matrix"] = dict(ms_per_step=solo["ms_per_step"], gbps=solo["gbps"],
                                                         frac_of_hbm_peak=solo["gbps"] / PEAK_HBM_GBPS,
                                                         launches_per_step=solo["launches_per_step"])
            extra["gemv_decode_m%d" % m] = best
        # the same decoder layer as dynamic-quant MatMuls (run-time input scale, fp32 out), gate and up as one launch
        # (mi_dynmm_run_group); beside it one launch per matrix, and the same rows on handles without the blocked
        # weight copy (2 rows and more then run on the GEMM tiles; one row needs no copy)
        for m in (1, 8):
            dyn = native_bench("dyndecode", m, 3, 500, 50, 0)
            if dyn and "gbps" in dyn:
                entry = dict(dyn, host="native C++ over the C ABI", bound="hbm", frac=dyn["gbps"] / PEAK_HBM_GBPS,
                             frac_of_hbm_peak=dyn["gbps"] / PEAK_HBM_GBPS)
                solo = native_bench("dyndecode", m, 3, 500, 50, 0, env={"NATIVE_BENCH_NO_GROUP": "1"})
                if solo and "gbps" in solo:
                    entry["one_launch_per_matrix"] = dict(ms_per_step=solo["ms_per_step"], gbps=solo["gbps"],
                                                          frac_of_hbm_peak=solo["gbps"] / PEAK_HBM_GBPS,
                                                          launches_per_step=solo["launches_per_step"])
                tiles = native_bench("dyndecode", m, 3, 200, 20, 1)
                if tiles and "gbps" in tiles:
                    entry["without_the_blocked_copy"] = dict(ms_per_step=tiles["ms_per_step"], gbps=tiles["gbps"])
                extra["dynmm_decode_m%d" % m] = entry
        warm = native_bench("warm", 1, 200, 20)
        if warm and "qkv" in warm:
            extra["gemv_m1_cache_warm"] = dict(warm, note="one matrix launched back to back: its weights stay in the "
                                               "256 MB Infinity Cache, so this is not an HBM figure")
        ceiling = (nread or {}).get("gbps") or (rd or {}).get("gbps")
        if ceiling and "gemv_decode_m1" in extra:
            extra["gemv_decode_m1"]["frac_of_read_stream"] = extra["gemv_decode_m1"]["gbps"] / ceiling
        extra.update(section("bert", lambda: bench_bert(max(100, args.steps), 3)) or {})
        extra.update(section("small_configs", lambda: bench_small_configs(max(200, args.steps), 20)) or {})
    result = {
        "metric": "int8 GEMM TOPS + % i8 MFMA peak; decode GEMV HBM GB/s; vs nnacl CPU",
        "value": g["tops"], "unit": "TOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": g["ms"], "ms_per_step_host_clock": g["host_ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "i8", "data": "synthetic",
        "config": {"workload": "config 5: int8 GEMM M=N=K=%d, per-channel requant to int8 (fused epilogue), zx=7, "
                               "int32 bias" % size,
                   "device_state": "settled: %d untimed launches (%.0f ms) from idle precede the warm-up, see "
                                   "settled_before_timing" % (g["settled"]["launches"], g["settled"]["ms"])},
        "settled_before_timing": g["settled"],
        "from_idle_before_settling": g["from_idle"],
        "roofline": {"bound": "mfma", "achieved": g["tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": g["tops"] / PEAK_INT8_TOPS, "traffic": None,
                     "kernel": HEADLINE_KERNEL, "ops_per_launch": g["ops"]},
    }
    tr = measured_traffic(args.workload)
    if tr:
        result["roofline"]["traffic"] = tr["bytes"]
        result["roofline"]["traffic_measured_at_commit"] = tr["commit"]
        result["roofline"]["traffic_measured_on_kernel"] = tr["kernel"]
        result["roofline"]["traffic_is_for_this_kernel"] = tr["kernel"] == HEADLINE_KERNEL
    if args.calibrate:
        L = lib.load_diag()
        src = torch.ones(256 << 20, dtype=torch.int8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            lib.check(L.mi_diag_copy(dst.data_ptr(), src.data_ptr(), 256 << 20, _stream()), "mi_diag_copy")
        torch.cuda.synchronize()
    if args.dynquant:
        from mindspore_amd import kernels as K
        from mindspore_amd import workloads as wl
        xq = torch.from_numpy(wl.bert_c3_activation(768)).cuda()
        dq = K.DynamicQuantKernel(False)
        for _ in range(100):
            dq.run(xq, fetch_params=False)
        torch.cuda.synchronize()
    if args.bert:
        from mindspore_amd import kernels as K
        from mindspore_amd import workloads as wl
        dq = K.DynamicQuantKernel(False)
        q, _ = dq.run(torch.from_numpy(wl.bert_c3_activation(768)).cuda(), fetch_params=False)
        for name, n, k in wl.BERT_SHAPES:
            wt = wl.bert_c3_weights(name, n, k)
            mm = K.MatmulDynamicInt8Kernel(wt["w"], wt["bias"], [K.QuantParam(float(sc), 0) for sc in wt["sw"]])
            qa = q if k == 768 else torch.randint(-128, 127, (4096, k), dtype=torch.int8, device="cuda")
            for _ in range(20):
                mm.run(qa, params_dev=dq.device_params())
        torch.cuda.synchronize()
    if args.c2:
        from mindspore_amd import kernels as K
        from mindspore_amd import workloads as wl
        x, layers = wl.mobilenet_c2()
        cur = torch.from_numpy(x).cuda()
        for L in layers:
            qp = [K.QuantParam(float(sc), int(z)) for sc, z in zip(L["sw"], L["zw"])]
            kern = K.ConvolutionInt8Kernel(L["w"], L["bias"], K.QuantParam(L["sx"], L["zx"]), qp,
                                           K.QuantParam(L["so"], L["zo"]), (L["stride"],) * 2, (1, 1), L["pad"],
                                           L["oc"] if L["kind"] == "dw" else 1, L["act"])
            for _ in range(20):
                nxt = kern.run(cur)
            cur = nxt
        torch.cuda.synchronize()
    if args.conv3x3:
        kern, xin, yout, _ = make_conv3x3()
        for _ in range(20):
            kern.run(xin, out=yout)
        torch.cuda.synchronize()
    if "mfma_only" in extra:
        # the matrix pipe alone on operands drawn like this GEMM's: the shader clock it sustains depends on the data
        lim = extra["mfma_only"]["uniform_int8_operands"]
        result["roofline"]["peak_on_this_data"] = lim["tops"]
        result["roofline"]["peak_on_this_data_clock_ghz"] = lim["shader_clock_ghz"]
        result["roofline"]["frac_of_peak_on_this_data"] = g["tops"] / lim["tops"]
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(g["case"], size)
        if not args.no_extra:
            cs = section("cpu_side_by_side", cpu_side_by_side)
            if cs:
                extra["cpu_side_by_side"] = cs
    extra["gemm%d_prepare_ms" % size] = g["prepare_ms"]
    if "host_path_ms" in g:
        extra["gemm%d_host_tensors" % size] = dict(ms=g["host_path_ms"], tops=g["ops"] / (g["host_path_ms"] * 1e-3) / 1e12,
                                                   note="mi_matmul_run_host: H2D + kernel + D2H, PCIe inclusive")
    if extra:
        result["extra"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
