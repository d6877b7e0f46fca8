// DynamicQuant, per tensor: fp32 -> int8 with scale / zero point taken from the tensor's min and max.
//   pass 1  dq_minmax   : one streaming read; per-lane running min/max with the strict </> updates of
//                         CalculateMinMaxFp32 (reference mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/
//                         dynamic_quant_int8.c:19-27; a NaN is never selected), wavefront shuffle reduction, one
//                         (min, max) partial per workgroup
//   pass 2  dq_quantize : every workgroup re-reduces the <= 256 partials (2 KiB, L2 resident), derives
//                         scale / zero point exactly as DynamicQuantCPUKernel::CalculatePerlayerScaleZp does
//                         (mindspore/lite/src/litert/kernel/cpu/int8/dynamic_quant.cc:156-186: float range, float
//                         division, zero point in double) and quantises its slice with the arithmetic of
//                         DoQuantizeFp32ToInt8 (.../nnacl/int8/quant_dtype_cast_int8.c:180-203: float reciprocal,
//                         float multiply, float add, round half away, clamp).  Workgroup 0 publishes the parameters.
// The second read of x (12.6 MB for the BERT activation) is served by L2 / Infinity Cache; no atomics, no third
// launch, results independent of scheduling.
#include <float.h>

#include "common.h"

namespace mi {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kDqThreads = 256;
constexpr int kDqElemsPerThread = 16;

__device__ __forceinline__ void upd(float v, float &lo, float &hi) {
  lo = v < lo ? v : lo;
  hi = v > hi ? v : hi;
}

template <int THREADS = 256>
__device__ __forceinline__ void block_minmax(float &lo, float &hi, float *slo, float *shi) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float l2 = __shfl_xor(lo, off), h2 = __shfl_xor(hi, off);
    lo = l2 < lo ? l2 : lo;
    hi = h2 > hi ? h2 : hi;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) {
    slo[wave] = lo;
    shi[wave] = hi;
  }
  __syncthreads();
  lo = slo[0];
  hi = shi[0];
#pragma unroll
  for (int w = 1; w < THREADS / 64; ++w) {
    lo = slo[w] < lo ? slo[w] : lo;
    hi = shi[w] > hi ? shi[w] : hi;
  }
  __syncthreads();
}

__global__ __launch_bounds__(kDqThreads) void dq_minmax_kernel(const float *__restrict__ x, int64_t n,
                                                               float2 *__restrict__ partials) {
  __shared__ float slo[kDqThreads / 64], shi[kDqThreads / 64];
  float lo = FLT_MAX, hi = -FLT_MAX;
  const int64_t stride = (int64_t)gridDim.x * kDqThreads;
  const int64_t gtid = (int64_t)blockIdx.x * kDqThreads + threadIdx.x;
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const int64_t n4 = n >> 2;
    const v4f *x4 = reinterpret_cast<const v4f *>(x);
    int64_t i = gtid;
    for (; i + 3 * stride < n4; i += 4 * stride) {  // four independent 16-byte loads in flight per thread
      v4f v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = x4[i + j * stride];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        upd(v[j].x, lo, hi);
        upd(v[j].y, lo, hi);
        upd(v[j].z, lo, hi);
        upd(v[j].w, lo, hi);
      }
    }
    for (; i < n4; i += stride) {
      const v4f v = x4[i];
      upd(v.x, lo, hi);
      upd(v.y, lo, hi);
      upd(v.z, lo, hi);
      upd(v.w, lo, hi);
    }
    for (int64_t i = (n4 << 2) + gtid; i < n; i += stride) upd(x[i], lo, hi);
  } else {
    for (int64_t i = gtid; i < n; i += stride) upd(x[i], lo, hi);
  }
  block_minmax(lo, hi, slo, shi);
  if (threadIdx.x == 0) partials[blockIdx.x] = make_float2(lo, hi);
}

__device__ __forceinline__ int double_to_int_x86(double r) {
  // cvttsd2si semantics: NaN or out of range -> INT_MIN
  return (r >= -2147483648.0 && r <= 2147483647.0) ? (int)r : INT32_MIN;
}

__device__ __forceinline__ int8_t quant_one(float v, float inv, float zpf) {
  if (v == INFINITY) return 127;
  if (v == -INFINITY) return -128;
  const float t = __fadd_rn(__fmul_rn(v, inv), zpf);
  const float r = roundf(t);  // half away from zero, exact
  int q = (r >= -2147483648.0f && r < 2147483648.0f) ? (int)r : INT32_MIN;
  q = q < 127 ? q : 127;
  q = q > -128 ? q : -128;
  return (int8_t)q;
}

// scale and zero point from the tensor's min and max (CalculatePerlayerScaleZp, dynamic_quant.cc:156-186)
__device__ __forceinline__ void scale_and_zp(float lo, float hi, int symmetric, float *scale_f, int *zp) {
  *zp = 0;
  if (!symmetric) {
    float range = __fsub_rn(hi, lo);
    if (range <= 0) range = 0.01f;
    *scale_f = __fdiv_rn(range, 255.0f);
    *zp = double_to_int_x86(round(-128.0 - (double)lo / (double)*scale_f));
  } else {
    const float a = fabsf(hi), b = fabsf(lo);
    const float big = (a < b) ? b : a;
    *scale_f = __fdiv_rn(__fmul_rn(2.0f, big), 254.0f);
  }
}

// Small tensors (a few activation rows: the decode step) in ONE launch of ONE workgroup: every thread keeps its up to
// 6 groups of four values in registers, the workgroup reduces min and max, derives the parameters and quantises from
// the registers.  The two-launch form costs such a tensor two launch latencies for a few microseconds of work
// (1 x 4096 values: 6.3 -> 4.2 us, 2 x 4096: 6.8 -> 4.9, 1 x 11008: 7.4 -> 5.1, 2 x 11008: 7.6 -> 7.0); from about
// 25 000 values on the arithmetic of a single CU takes longer than the second launch (8 x 4096: 9.0 against 7.5 us).
constexpr int kDqSingleThreads = 1024;
constexpr int kDqSingleGroups = 6;  // float4 groups per thread: up to 24576 values
__global__ __launch_bounds__(kDqSingleThreads) void dq_single_kernel(const float *__restrict__ x, int n, int symmetric,
                                                                     mi_dq_params *__restrict__ params,
                                                                     int8_t *__restrict__ q) {
  __shared__ float slo[kDqSingleThreads / 64], shi[kDqSingleThreads / 64];
  const int tid = threadIdx.x, n4 = n >> 2;
  const v4f *x4 = reinterpret_cast<const v4f *>(x);  // (the host checked the alignment)
  v4f v[kDqSingleGroups];
  float lo = FLT_MAX, hi = -FLT_MAX;
#pragma unroll
  for (int j = 0; j < kDqSingleGroups; ++j) {
    const int i = tid + j * kDqSingleThreads;
    if (i < n4) {
      v[j] = x4[i];
      upd(v[j].x, lo, hi);
      upd(v[j].y, lo, hi);
      upd(v[j].z, lo, hi);
      upd(v[j].w, lo, hi);
    }
  }
  float tail = 0.0f;  // the up to three values past the last whole group
  const int ti = (n4 << 2) + tid;
  if (ti < n) {
    tail = x[ti];
    upd(tail, lo, hi);
  }
  block_minmax<kDqSingleThreads>(lo, hi, slo, shi);
  float scale_f;
  int zp;
  scale_and_zp(lo, hi, symmetric, &scale_f, &zp);
  if (tid == 0) {
    params->scale = (double)scale_f;
    params->scale_f = scale_f;
    params->zero_point = zp;
    params->real_min = lo;
    params->real_max = hi;
  }
  const float inv = __fdiv_rn(1.0f, scale_f);
  const float zpf = (float)zp;
#pragma unroll
  for (int j = 0; j < kDqSingleGroups; ++j) {
    const int i = tid + j * kDqSingleThreads;
    if (i < n4) {
      union {
        int w;
        int8_t b[4];
      } u;
      u.b[0] = quant_one(v[j].x, inv, zpf);
      u.b[1] = quant_one(v[j].y, inv, zpf);
      u.b[2] = quant_one(v[j].z, inv, zpf);
      u.b[3] = quant_one(v[j].w, inv, zpf);
      reinterpret_cast<int *>(q)[i] = u.w;
    }
  }
  if (ti < n) q[ti] = quant_one(tail, inv, zpf);
}

__global__ __launch_bounds__(kDqThreads) void dq_quantize_kernel(const float *__restrict__ x, int64_t n,
                                                                 int symmetric,
                                                                 const float2 *__restrict__ partials, int nparts,
                                                                 mi_dq_params *__restrict__ params,
                                                                 int8_t *__restrict__ q) {
  __shared__ float slo[kDqThreads / 64], shi[kDqThreads / 64];
  // request this thread's 16 values first: they arrive while the partials are reduced and the scale is derived
  const int64_t base = ((int64_t)blockIdx.x * kDqThreads + threadIdx.x) * kDqElemsPerThread;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) & 15) == 0) && ((reinterpret_cast<uintptr_t>(q) & 15) == 0);
  const bool fast = aligned && base + kDqElemsPerThread <= n;
  v4f xv[4];
  {
    // never predicated: a thread without a full group of its own re-reads the first one (n >= 16 on this path)
    const int64_t safe = fast ? base : 0;
    const v4f *x4 = reinterpret_cast<const v4f *>(x + (aligned && n >= kDqElemsPerThread ? safe : 0));
    if (aligned && n >= kDqElemsPerThread) {
#pragma unroll
      for (int j = 0; j < 4; ++j) xv[j] = x4[j];
    }
  }

  float lo = FLT_MAX, hi = -FLT_MAX;
  for (int i = threadIdx.x; i < nparts; i += kDqThreads) {
    const float2 p = partials[i];
    lo = p.x < lo ? p.x : lo;
    hi = p.y > hi ? p.y : hi;
  }
  block_minmax(lo, hi, slo, shi);

  float scale_f;
  int zp;
  scale_and_zp(lo, hi, symmetric, &scale_f, &zp);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    params->scale = (double)scale_f;
    params->scale_f = scale_f;
    params->zero_point = zp;
    params->real_min = lo;
    params->real_max = hi;
  }
  const float inv = __fdiv_rn(1.0f, scale_f);
  const float zpf = (float)zp;

  if (base >= n) return;
  if (fast) {
    union {
      int4 v;
      int8_t b[16];
    } u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const v4f v = xv[j];
      u.b[4 * j + 0] = quant_one(v.x, inv, zpf);
      u.b[4 * j + 1] = quant_one(v.y, inv, zpf);
      u.b[4 * j + 2] = quant_one(v.z, inv, zpf);
      u.b[4 * j + 3] = quant_one(v.w, inv, zpf);
    }
    *reinterpret_cast<int4 *>(q + base) = u.v;
  } else {
    const int64_t end = base + kDqElemsPerThread < n ? base + kDqElemsPerThread : n;
    for (int64_t i = base; i < end; ++i) q[i] = quant_one(x[i], inv, zpf);
  }
}

// DynamicQuant with preferred axes (one scale / zero point per segment): after the preferred axes lead, the tensor is
// `segments` contiguous runs of `unit` elements (DynamicQuantCPUKernel::ReSize / CalculateMinMax / QuantData,
// mindspore/lite/src/litert/kernel/cpu/int8/dynamic_quant.cc:59-94,118-143,236-246; scale and zero point per segment
// as CalculatePerChannelScaleZp :188-218, the same formulas as the per-tensor case).  One wave per segment: first
// sweep min/max, second sweep (the run is L1/L2 resident by then) quantises.
__global__ __launch_bounds__(kDqThreads) void dq_segments_kernel(const float *__restrict__ x, int64_t segments,
                                                                 int64_t unit, int symmetric,
                                                                 mi_dq_params *__restrict__ params,
                                                                 int8_t *__restrict__ q) {
  const int lane = threadIdx.x & 63;
  const int64_t seg = (int64_t)blockIdx.x * (kDqThreads / 64) + (threadIdx.x >> 6);
  if (seg >= segments) return;
  const float *xs = x + seg * unit;
  int8_t *qs = q + seg * unit;
  const bool vec = ((reinterpret_cast<uintptr_t>(xs) & 15) == 0) && ((reinterpret_cast<uintptr_t>(qs) & 3) == 0);
  const int64_t n4 = vec ? unit >> 2 : 0;
  float lo = FLT_MAX, hi = -FLT_MAX;
  const v4f *x4 = reinterpret_cast<const v4f *>(xs);
  for (int64_t i = lane; i < n4; i += 64) {
    const v4f v = x4[i];
    upd(v.x, lo, hi);
    upd(v.y, lo, hi);
    upd(v.z, lo, hi);
    upd(v.w, lo, hi);
  }
  for (int64_t i = (n4 << 2) + lane; i < unit; i += 64) upd(xs[i], lo, hi);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float l2 = __shfl_xor(lo, off), h2 = __shfl_xor(hi, off);
    lo = l2 < lo ? l2 : lo;
    hi = h2 > hi ? h2 : hi;
  }
  float scale_f;
  double scale_d;
  int zp = 0;
  if (!symmetric) {
    float range = __fsub_rn(hi, lo);
    if (range <= 0) range = 0.01f;
    scale_f = __fdiv_rn(range, 255.0f);
    scale_d = (double)scale_f;
    zp = double_to_int_x86(round(-128.0 - (double)lo / scale_d));
  } else {
    const float a = fabsf(hi), b = fabsf(lo);
    const float big = (a < b) ? b : a;
    scale_f = __fdiv_rn(__fmul_rn(2.0f, big), 254.0f);
    scale_d = (double)scale_f;
  }
  if (lane == 0) {
    mi_dq_params *p = params + seg;
    p->scale = scale_d;
    p->scale_f = scale_f;
    p->zero_point = zp;
    p->real_min = lo;
    p->real_max = hi;
  }
  const float inv = __fdiv_rn(1.0f, scale_f);
  const float zpf = (float)zp;
  for (int64_t i = lane; i < n4; i += 64) {
    const v4f v = x4[i];
    union {
      int w;
      int8_t b[4];
    } u;
    u.b[0] = quant_one(v.x, inv, zpf);
    u.b[1] = quant_one(v.y, inv, zpf);
    u.b[2] = quant_one(v.z, inv, zpf);
    u.b[3] = quant_one(v.w, inv, zpf);
    *reinterpret_cast<int *>(qs + 4 * i) = u.w;
  }
  for (int64_t i = (n4 << 2) + lane; i < unit; i += 64) qs[i] = quant_one(xs[i], inv, zpf);
}

int launch_dynquant_segments(const float *x, int64_t segments, int64_t unit, int symmetric, mi_dq_params *params,
                             int8_t *q, hipStream_t stream) {
  const int64_t blocks = (segments + kDqThreads / 64 - 1) / (kDqThreads / 64);
  if (blocks > 0x7fffffff) {
    set_error("dynquant: too many segments");
    return MI_PARAM_INVALID;
  }
  hipLaunchKernelGGL(dq_segments_kernel, dim3((unsigned)blocks), dim3(kDqThreads), 0, stream, x, segments, unit,
                     symmetric, params, q);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

int launch_dynquant(const float *x, int64_t n, int symmetric, float2 *partials, mi_dq_params *params, int8_t *q,
                    hipStream_t stream) {
  if (n <= (int64_t)kDqSingleThreads * kDqSingleGroups * 4 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(q) & 3) == 0) {
    hipLaunchKernelGGL(dq_single_kernel, dim3(1), dim3(kDqSingleThreads), 0, stream, x, (int)n, symmetric, params, q);
    MI_HIP_CHECK(hipGetLastError());
    return MI_OK;
  }
  const int64_t per_block = (int64_t)kDqThreads * kDqElemsPerThread;
  int64_t want = (n + per_block - 1) / per_block;
  // pass 1: at most one workgroup per partial a thread of pass 2 reads in a single step
  const int64_t want1 = (want + 2) / 3;
  const int nparts = (int)(want1 < 1 ? 1 : (want1 > kDqThreads ? kDqThreads : want1));
  hipLaunchKernelGGL(dq_minmax_kernel, dim3(nparts), dim3(kDqThreads), 0, stream, x, n, partials);
  MI_HIP_CHECK(hipGetLastError());
  const int64_t qblocks = want < 1 ? 1 : want;
  if (qblocks > 0x7fffffff) {
    set_error("dynquant: tensor too large");
    return MI_PARAM_INVALID;
  }
  hipLaunchKernelGGL(dq_quantize_kernel, dim3((unsigned)qblocks), dim3(kDqThreads), 0, stream, x, n, symmetric,
                     partials, nparts, params, q);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

}  // namespace mi
