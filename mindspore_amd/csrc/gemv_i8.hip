// Skinny-M (decode) int8 GEMV with the requantising epilogue of the full-quant MatMul: M <= 8 activation rows
// against an [n_pad][k_pad] int8 weight matrix.  The kernel is HBM-bound on the weight stream, so the design goal
// is "every weight byte crosses HBM once, in 1 KiB coalesced wave loads, with enough loads in flight":
//   - a wave owns R consecutive output channels and walks K in 1 KiB segments (64 lanes x 16 bytes);
//   - it keeps two groups of U segments x R rows of 16-byte loads in flight (software prefetch);
//   - the M activation rows are staged once per workgroup in LDS and re-read as 16-byte fragments;
//   - products use v_dot4_i32_i8; the K reduction across lanes happens once at the end.
// Arithmetic reference: MatmulInt8Opt, mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/matmul_int8.c:296-331.
#include "common.h"
#include "quant_math.h"

namespace mi {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__device__ __forceinline__ int dot16(v4i w, v4i a, int acc) {
  acc = __builtin_amdgcn_sdot4(w.x, a.x, acc, false);
  acc = __builtin_amdgcn_sdot4(w.y, a.y, acc, false);
  acc = __builtin_amdgcn_sdot4(w.z, a.z, acc, false);
  acc = __builtin_amdgcn_sdot4(w.w, a.w, acc, false);
  return acc;
}

struct GemvArgs {
  const int8_t *a;
  int64_t lda;
  int kchunks;  // K / 16
  const int8_t *w;
  int ldw;  // k_pad
  int n;
  int8_t *c;
  int64_t ldc;
};

template <int M, int R, int U>
__global__ __launch_bounds__(256) void gemv_i8_kernel(GemvArgs g, RequantParams rq) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  v4i *sa = reinterpret_cast<v4i *>(smem);  // [M][kchunks]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_base = (blockIdx.x * 4 + wave) * R;
  const int nseg = (g.kchunks + 63) >> 6;
  const int ngroups = (nseg + U - 1) / U;
  const int8_t *wrow = g.w + (int64_t)n_base * g.ldw;

  v4i wcur[U][R], wnext[U][R];
  auto load_group = [&](v4i(&dst)[U][R], int grp) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int chunk = (grp * U + u) * 64 + lane;
      const bool valid = chunk < g.kchunks;
#pragma unroll
      for (int rr = 0; rr < R; ++rr) {
        v4i z = {0, 0, 0, 0};
        dst[u][rr] = valid ? *reinterpret_cast<const v4i *>(wrow + (int64_t)rr * g.ldw + (int64_t)chunk * 16) : z;
      }
    }
  };
  load_group(wcur, 0);

  // stage the activations
  for (int idx = tid; idx < M * g.kchunks; idx += 256) {
    const int m = idx / g.kchunks, ch = idx - m * g.kchunks;
    sa[idx] = *reinterpret_cast<const v4i *>(g.a + (int64_t)m * g.lda + (int64_t)ch * 16);
  }
  __syncthreads();

  int acc[R][M];
  int asum[M];
#pragma unroll
  for (int rr = 0; rr < R; ++rr)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[rr][m] = 0;
#pragma unroll
  for (int m = 0; m < M; ++m) asum[m] = 0;

  for (int grp = 0; grp < ngroups; ++grp) {
    if (grp + 1 < ngroups) load_group(wnext, grp + 1);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int chunk = (grp * U + u) * 64 + lane;
      if (chunk < g.kchunks) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const v4i af = sa[m * g.kchunks + chunk];
          if (rq.has_zw) {
            v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
            asum[m] = dot16(af, ones, asum[m]);
          }
#pragma unroll
          for (int rr = 0; rr < R; ++rr) acc[rr][m] = dot16(wcur[u][rr], af, acc[rr][m]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rr = 0; rr < R; ++rr) wcur[u][rr] = wnext[u][rr];
  }

  // reduce over lanes; afterwards every lane holds every total and lane rr*M + m finishes output (m, n_base + rr)
  int mine = 0, my_asum = 0;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    int s = 0;
    if (rq.has_zw) s = wave_sum(asum[m]);
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
      const int t = wave_sum(acc[rr][m]);
      if (lane == rr * M + m) {
        mine = t;
        my_asum = s;
      }
    }
  }
  if (lane < R * M) {
    const int rr = lane / M, m = lane - rr * M;
    const int n = n_base + rr;
    if (n < g.n) {
      uint32_t v = (uint32_t)mine;
      if (rq.has_zw) v -= (uint32_t)my_asum * (uint32_t)rq.zw[n];
      v += (uint32_t)rq.bias2[n];
      const int32_t mult = rq.mult[n], e = rq.rshift[n];
      int32_t y;
      if (rq.fast) {
        y = rdiv_pot_fast(srdhm_nosat((int32_t)v, mult), e, (1 << e) >> 1);
      } else {
        y = rdiv_pot(srdhm((int32_t)(v << rq.lshift[n]), mult), e);
      }
      y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
      y = y < rq.amax ? y : rq.amax;
      y = y > rq.amin ? y : rq.amin;
      g.c[(int64_t)m * g.ldc + n] = (int8_t)y;
    }
  }
}

template <int M, int R>
static int launch_mr(const GemvArgs &g, const RequantParams &rq, hipStream_t stream) {
  constexpr int U = 2;
  auto kern = gemv_i8_kernel<M, R, U>;
  const int lds_bytes = M * g.kchunks * 16;
  if (lds_bytes > 64 * 1024) {
    static bool attr_set = false;
    if (!attr_set) {
      MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      attr_set = true;
    }
  }
  const int rows_per_block = 4 * R;
  const int blocks = (g.n + rows_per_block - 1) / rows_per_block;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds_bytes, stream, g, rq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int M>
static int launch_m(const GemvArgs &g, const RequantParams &rq, hipStream_t stream) {
  // fewer rows per wave when there are few output channels, so that every CU still gets several waves
  if (g.n <= 8192) return launch_mr<M, 2>(g, rq, stream);
  return launch_mr<M, 4>(g, rq, stream);
}

int launch_gemv_requant(const int8_t *a, int64_t lda, int m, int k, const int8_t *w, int k_pad, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream) {
  if (a == nullptr || w == nullptr || c == nullptr) {
    set_error("gemv: null pointer");
    return MI_NULL_PTR;
  }
  if (m < 1 || m > kGemvMaxRows || n <= 0 || k <= 0 || (k & 15) != 0 || (lda & 15) != 0 || lda < k ||
      k_pad % kKPad != 0 || k_pad < k || (reinterpret_cast<uintptr_t>(a) & 15) != 0 ||
      (int64_t)m * k > 160 * 1024 - 1024) {
    set_error("gemv: unsupported operand geometry m=%d n=%d k=%d lda=%lld", m, n, k, (long long)lda);
    return MI_PARAM_INVALID;
  }
  GemvArgs g{a, lda, k / 16, w, k_pad, n, c, ldc};
  switch (m) {
    case 1: return launch_m<1>(g, rq, stream);
    case 2: return launch_m<2>(g, rq, stream);
    case 3: return launch_m<3>(g, rq, stream);
    case 4: return launch_m<4>(g, rq, stream);
    case 5: return launch_m<5>(g, rq, stream);
    case 6: return launch_m<6>(g, rq, stream);
    case 7: return launch_m<7>(g, rq, stream);
    default: return launch_m<8>(g, rq, stream);
  }
}

}  // namespace mi
