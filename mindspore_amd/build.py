"""Builds libmi355x_int8.so (HIP kernels + C ABI) for gfx950 with hipcc.  Cross-compiles without a GPU."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmi355x_int8.so")
DIAG_LIB = os.path.join(HERE, "libmi355x_diag.so")  # the benchmark's measurement aids, not part of the product
NATIVE_BENCH = os.path.join(HERE, "native_bench")
SOURCES = ["capi.hip", "gemm_i8.hip", "gemv_i8.hip", "conv_i8.hip", "dynquant.hip", "infer_shape.hip"]
# -ffp-contract=off: the float steps of DynamicQuant / dynamic MatMul and the host-side multiplier derivation are
# separately rounded operations in the reference and must not be fused.
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]


def build_library(verbose=False):
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        if verbose or p.returncode != 0:
            print(" ".join(cmd))
            print(out)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed for %s" % cmd[-3])
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(link)
    subprocess.check_call(["hipcc"] + FLAGS + ["-shared", os.path.join(CSRC, "diag.hip"), "-o", DIAG_LIB])
    # the native benchmark host (a C++ caller of the C ABI, like a provider kernel)
    subprocess.check_call(["hipcc", "-O2", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", "-Wno-unused-result",
                           os.path.join(CSRC, "native_bench.cc"), "-o", NATIVE_BENCH, "-L" + HERE, "-lmi355x_int8", "-lmi355x_diag",
                           "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
