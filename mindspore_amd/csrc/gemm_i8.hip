// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8) with fused epilogues:
//   EPI_REQUANT : + folded bias, - zw * input-row-sum, fixed-point requantise, + zo, clamp  -> int8
//                 (the arithmetic of MatmulInt8Opt / MatMulInt8_8x8_r, reference
//                  mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/matmul_int8.c:296-364)
//   EPI_DEQUANT : zero-point corrections, (sx*sw) * (float)acc, + bias, activation         -> fp32
//                 (DynamicMatmul4x16x4AIWI, .../nnacl/int8/dynamic_matmul_int8.c:99-143)
//
// Data movement.  Both operands are K-contiguous: activations A[M][K] and packed weights W[n_pad][k_pad].  A
// workgroup owns a TILE_M x TILE_N output tile and walks K in steps of 128 bytes.  Each step stages
// (TILE_M + TILE_N) rows x 128 B in LDS (double buffered); a row is eight 16-byte chunks and chunk c of row r is
// stored at slot c ^ ((r >> 1) & 7), which makes both the 16-byte stores of the loader and the 16-byte operand
// reads of the MFMA loop bank-conflict free.  The weight tile is the MFMA "A" operand (its rows are output
// channels) and the activation tile the "B" operand, so a lane ends up holding 4 consecutive output channels of
// one output row: the epilogue packs them into one 32-bit store, and the input-row sum a lane needs is the one it
// accumulated itself from its activation fragments (v_dot4 against 0x01010101).
#include "common.h"
#include "quant_math.h"

namespace mi {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int BK = 128;  // bytes of K per LDS stage
enum { EPI_REQUANT = 0, EPI_DEQUANT = 1 };

__device__ __forceinline__ int lds_slot(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

struct GemmArgs {
  const int8_t *a;
  int64_t lda;
  int m;
  int kchunks;  // valid 16-byte chunks per activation row (K / 16)
  const int8_t *w;
  int ldw;     // k_pad
  int ktiles;  // k_pad / 128
  int n;
  int tiles_m, tiles_n;
  void *c;
  int64_t ldc;
};

template <int TILE_N, int TILE_M, int WAVES_N, int WAVES_M, int EPI, bool HAS_ZW, bool FAST>
__global__ __launch_bounds__(WAVES_N *WAVES_M * 64) void gemm_i8_kernel(GemmArgs g, RequantParams rq,
                                                                         DequantParams dq) {
  constexpr int THREADS = WAVES_N * WAVES_M * 64;
  constexpr int WN = TILE_N / WAVES_N, WM = TILE_M / WAVES_M;
  constexpr int TN = WN / 32, TM = WM / 32;
  constexpr int W_CHUNKS = TILE_N * 8 / THREADS, A_CHUNKS = TILE_M * 8 / THREADS;
  constexpr int ROWS_PER_PASS = THREADS / 8;
  constexpr int STAGE_BYTES = (TILE_N + TILE_M) * BK;
  static_assert(W_CHUNKS >= 1 && A_CHUNKS >= 1, "tile too small for the thread count");

  extern __shared__ __attribute__((aligned(16))) char smem[];

  // ---- tile assignment: hardware deals consecutive workgroup ids round-robin over the 8 XCDs (each with its own
  //      L2), so ids that share an XCD are mapped to a compact block of tiles, 4 tiles tall ----
  int id = blockIdx.x;
  {
    const int nb = gridDim.x, per = nb >> 3;
    if (id < per * 8) id = (id & 7) * per + (id >> 3);
  }
  int tile_m, tile_n;
  {
    constexpr int G = 4;
    const int width = G * g.tiles_n;
    const int group = id / width, first = group * G;
    const int gsize = min(g.tiles_m - first, G);
    tile_m = first + (id % width) % gsize;
    tile_n = (id % width) / gsize;
  }
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wn = wave % WAVES_N, wm = wave / WAVES_N;
  const int r = lane & 31, h = lane >> 5;

  // ---- loader: thread t moves chunk (t & 7) of rows (t >> 3) + i * ROWS_PER_PASS ----
  const int lc = tid & 7, lrow = tid >> 3;
  v4i wreg[W_CHUNKS], areg[A_CHUNKS];
  const int8_t *wsrc = g.w + (int64_t)(n0 + lrow) * g.ldw + lc * 16;
  const int8_t *asrc[A_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    int m = m0 + lrow + i * ROWS_PER_PASS;
    m = m < g.m ? m : g.m - 1;
    asrc[i] = g.a + (int64_t)m * g.lda + lc * 16;
  }
  auto load_tile = [&](int kt) {
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i)
      wreg[i] = *reinterpret_cast<const v4i *>(wsrc + (int64_t)i * ROWS_PER_PASS * g.ldw + kt * BK);
    const bool valid = kt * 8 + lc < g.kchunks;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      v4i z = {0, 0, 0, 0};
      areg[i] = valid ? *reinterpret_cast<const v4i *>(asrc[i] + kt * BK) : z;
    }
  };
  auto store_tile = [&](int stage) {
    char *sw = smem + stage * STAGE_BYTES;
    char *sa = sw + TILE_N * BK;
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int row = lrow + i * ROWS_PER_PASS;
      *reinterpret_cast<v4i *>(sw + row * BK + (lds_slot(row, lc) << 4)) = wreg[i];
    }
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int row = lrow + i * ROWS_PER_PASS;
      *reinterpret_cast<v4i *>(sa + row * BK + (lds_slot(row, lc) << 4)) = areg[i];
    }
  };

  v16i acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
  int rowsum[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) rowsum[j] = 0;

  const int frag_swz = (r >> 1) & 7;  // rows handled by this lane are r + multiples of 32
  const int w_row0 = wn * WN + r, a_row0 = wm * WM + r;

  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < g.ktiles; ++kt) {
    const bool more = kt + 1 < g.ktiles;
    if (more) load_tile(kt + 1);
    const char *sw = smem + (kt & 1) * STAGE_BYTES;
    const char *sa = sw + TILE_N * BK;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int slot = ((2 * s + h) ^ frag_swz) << 4;
      v4i wf[TN], af[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) wf[i] = *reinterpret_cast<const v4i *>(sw + (w_row0 + i * 32) * BK + slot);
#pragma unroll
      for (int j = 0; j < TM; ++j) af[j] = *reinterpret_cast<const v4i *>(sa + (a_row0 + j * 32) * BK + slot);
      if (HAS_ZW) {
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          int t = rowsum[j];
          t = __builtin_amdgcn_sdot4(af[j].x, 0x01010101, t, false);
          t = __builtin_amdgcn_sdot4(af[j].y, 0x01010101, t, false);
          t = __builtin_amdgcn_sdot4(af[j].z, 0x01010101, t, false);
          t = __builtin_amdgcn_sdot4(af[j].w, 0x01010101, t, false);
          rowsum[j] = t;
        }
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], af[j], acc[i][j], 0, 0, 0);
    }
    if (more) store_tile((kt + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue.  acc[i][j][4*q + e] is output channel n0 + wn*WN + 32*i + 8*q + 4*h + e of output row
  //      m0 + wm*WM + 32*j + r ----
  if (HAS_ZW) {
#pragma unroll
    for (int j = 0; j < TM; ++j) rowsum[j] += __shfl_xor(rowsum[j], 32);
  }

  if (EPI == EPI_REQUANT) {
    int8_t *c = static_cast<int8_t *>(g.c);
    const bool vec_ok = ((g.n & 3) == 0) && ((g.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(c) & 3) == 0);
#pragma unroll
    for (int i = 0; i < TN; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nb = n0 + wn * WN + i * 32 + q * 8 + h * 4;
        if (nb >= g.n) continue;
        const v4i mult4 = *reinterpret_cast<const v4i *>(rq.mult + nb);
        const v4i bias4 = *reinterpret_cast<const v4i *>(rq.bias2 + nb);
        const v4i e4 = *reinterpret_cast<const v4i *>(rq.rshift + nb);
        v4i zw4 = {0, 0, 0, 0}, ls4 = {0, 0, 0, 0}, half4 = {0, 0, 0, 0};
        if (HAS_ZW) zw4 = *reinterpret_cast<const v4i *>(rq.zw + nb);
        if (!FAST) ls4 = *reinterpret_cast<const v4i *>(rq.lshift + nb);
        if (FAST) {
#pragma unroll
          for (int e = 0; e < 4; ++e) half4[e] = (1 << e4[e]) >> 1;
        }
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const int m = m0 + wm * WM + j * 32 + r;
          uint32_t packed = 0;
          int8_t bytes[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            uint32_t v = (uint32_t)acc[i][j][q * 4 + e];
            if (HAS_ZW) v -= (uint32_t)rowsum[j] * (uint32_t)zw4[e];
            v += (uint32_t)bias4[e];
            int32_t y;
            if (FAST) {
              y = rdiv_pot_fast(srdhm_nosat((int32_t)v, mult4[e]), e4[e], half4[e]);
            } else {
              y = rdiv_pot(srdhm((int32_t)(v << ls4[e]), mult4[e]), e4[e]);
            }
            y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
            y = y < rq.amax ? y : rq.amax;
            y = y > rq.amin ? y : rq.amin;
            bytes[e] = (int8_t)y;
            packed |= ((uint32_t)y & 0xffu) << (8 * e);
          }
          if (m < g.m) {
            int8_t *dst = c + (int64_t)m * g.ldc + nb;
            if (vec_ok) {
              *reinterpret_cast<uint32_t *>(dst) = packed;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (nb + e < g.n) dst[e] = bytes[e];
            }
          }
        }
      }
    }
  } else {
    float *c = static_cast<float *>(g.c);
    const bool vec_ok = ((g.n & 3) == 0) && ((g.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
    float sx = dq.sx;
    int32_t zx = dq.zx;
    if (dq.qp_dev != nullptr) {
      sx = dq.qp_dev->scale_f;
      zx = dq.qp_dev->zero_point;
    }
    const uint32_t kzz = (uint32_t)dq.deep * (uint32_t)zx * (uint32_t)dq.zw0;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nb = n0 + wn * WN + i * 32 + q * 8 + h * 4;
        if (nb >= g.n) continue;
        const v4f ws4 = *reinterpret_cast<const v4f *>(dq.wscale + nb);
        const v4i wsum4 = *reinterpret_cast<const v4i *>(dq.wsum + nb);
        v4f b4 = {0.f, 0.f, 0.f, 0.f};
        if (dq.bias != nullptr) b4 = *reinterpret_cast<const v4f *>(dq.bias + nb);
        float ms[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) ms[e] = __fmul_rn(sx, ws4[e]);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const int m = m0 + wm * WM + j * 32 + r;
          v4f o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            uint32_t v = (uint32_t)acc[i][j][q * 4 + e];
            if (HAS_ZW) v -= (uint32_t)dq.zw0 * (uint32_t)rowsum[j];
            v -= (uint32_t)zx * (uint32_t)wsum4[e];
            v += kzz;
            float d = __fmul_rn(ms[e], (float)(int32_t)v);
            if (dq.bias != nullptr) d = __fadd_rn(d, b4[e]);
            if (dq.act == MI_ACT_RELU) {
              d = (0.0f > d) ? 0.0f : d;
            } else if (dq.act == MI_ACT_RELU6) {
              d = (0.0f > d) ? 0.0f : d;
              d = (6.0f < d) ? 6.0f : d;
            }
            o[e] = d;
          }
          if (m < g.m) {
            float *dst = c + (int64_t)m * g.ldc + nb;
            if (vec_ok) {
              *reinterpret_cast<v4f *>(dst) = o;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (nb + e < g.n) dst[e] = o[e];
            }
          }
        }
      }
    }
  }
}

// ---- host side -----------------------------------------------------------------------------------------------
template <int TILE_N, int TILE_M, int EPI, bool HAS_ZW, bool FAST>
static int launch_cfg(GemmArgs g, const RequantParams &rq, const DequantParams &dq, hipStream_t stream) {
  constexpr int WAVES_N = 2, WAVES_M = 2;
  auto kern = gemm_i8_kernel<TILE_N, TILE_M, WAVES_N, WAVES_M, EPI, HAS_ZW, FAST>;
  constexpr int lds_bytes = 2 * (TILE_N + TILE_M) * BK;
  static bool attr_set = false;  // benign race: idempotent
  if (!attr_set) {
    MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     lds_bytes));
    attr_set = true;
  }
  g.tiles_m = (g.m + TILE_M - 1) / TILE_M;
  g.tiles_n = (g.n + TILE_N - 1) / TILE_N;
  const int blocks = g.tiles_m * g.tiles_n;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(WAVES_N * WAVES_M * 64), lds_bytes, stream, g, rq, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int EPI, bool HAS_ZW, bool FAST>
static int launch_pick_tile(const GemmArgs &g, const RequantParams &rq, const DequantParams &dq,
                            hipStream_t stream) {
  const int64_t tiles_l = (int64_t)((g.m + 255) / 256) * ((g.n + 255) / 256);
  const int64_t tiles_m = (int64_t)((g.m + 127) / 128) * ((g.n + 127) / 128);
  if (tiles_l >= 192) return launch_cfg<256, 256, EPI, HAS_ZW, FAST>(g, rq, dq, stream);
  if (tiles_m >= 128) return launch_cfg<128, 128, EPI, HAS_ZW, FAST>(g, rq, dq, stream);
  return launch_cfg<64, 64, EPI, HAS_ZW, FAST>(g, rq, dq, stream);
}

static int check_args(const int8_t *a, int64_t lda, int m, int k, const int8_t *w, int k_pad, int n, const void *c) {
  if (a == nullptr || w == nullptr || c == nullptr) {
    set_error("gemm: null pointer");
    return MI_NULL_PTR;
  }
  if (m <= 0 || n <= 0 || k <= 0 || (k & 15) != 0 || (lda & 15) != 0 || lda < k || k_pad % kKPad != 0 || k_pad < k ||
      (reinterpret_cast<uintptr_t>(a) & 15) != 0) {
    set_error("gemm: unsupported operand geometry m=%d n=%d k=%d lda=%lld k_pad=%d", m, n, k, (long long)lda, k_pad);
    return MI_PARAM_INVALID;
  }
  return MI_OK;
}

int launch_gemm_requant(const int8_t *a, int64_t lda, int m, int k, const int8_t *w, int k_pad, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream) {
  int rc = check_args(a, lda, m, k, w, k_pad, n, c);
  if (rc != MI_OK) return rc;
  GemmArgs g{a, lda, m, k / 16, w, k_pad, k_pad / BK, n, 0, 0, c, ldc};
  DequantParams dq{};
  if (rq.has_zw) {
    return rq.fast ? launch_pick_tile<EPI_REQUANT, true, true>(g, rq, dq, stream)
                   : launch_pick_tile<EPI_REQUANT, true, false>(g, rq, dq, stream);
  }
  return rq.fast ? launch_pick_tile<EPI_REQUANT, false, true>(g, rq, dq, stream)
                 : launch_pick_tile<EPI_REQUANT, false, false>(g, rq, dq, stream);
}

int launch_gemm_dequant(const int8_t *a, int64_t lda, int m, int k, const int8_t *w, int k_pad, int n,
                        const DequantParams &dq, float *c, int64_t ldc, hipStream_t stream) {
  int rc = check_args(a, lda, m, k, w, k_pad, n, c);
  if (rc != MI_OK) return rc;
  GemmArgs g{a, lda, m, k / 16, w, k_pad, k_pad / BK, n, 0, 0, c, ldc};
  RequantParams rq{};
  return dq.zw0 != 0 ? launch_pick_tile<EPI_DEQUANT, true, false>(g, rq, dq, stream)
                     : launch_pick_tile<EPI_DEQUANT, false, false>(g, rq, dq, stream);
}

}  // namespace mi
