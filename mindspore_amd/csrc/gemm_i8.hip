// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8) with fused epilogues:
//   EPI_REQUANT : + folded bias, - zw * input-row-sum, fixed-point requantise, + zo, clamp  -> int8
//                 (the arithmetic of MatmulInt8Opt / MatMulInt8_8x8_r, reference
//                  mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/matmul_int8.c:296-364)
//   EPI_DEQUANT : zero-point corrections, (sx*sw) * (float)acc, + bias, activation         -> fp32
//                 (DynamicMatmul4x16x4AIWI, .../nnacl/int8/dynamic_matmul_int8.c:99-143)
//
// Both operands are K-contiguous: activations A[M][K] and packed weights W[n_pad][k_pad].  A workgroup of four
// waves (2 x 2) owns a TILE_M x TILE_N output tile; the weight tile is the MFMA "A" operand (its rows are output
// channels) and the activation tile the "B" operand, so a lane ends up holding 4 consecutive output channels of
// one output row: the epilogue packs them into one 32-bit store, per-channel parameters are 16-byte loads, and
// the input-row sum a lane needs is the one it accumulated itself (v_dot4 against 0x01010101).
//
// Two main loops, both moving tiles global -> LDS with asynchronous 16-byte-per-lane loads and reading operand
// fragments for the next K sub-step from LDS while the MFMAs of the current one run:
//   * K blocks of 128 bytes (gemm_kblock_body): whole cache lines per load, five LDS slots, one barrier per block;
//     256 x 256 tiles with one workgroup per CU for the large compute-bound shapes, 128 x 128 tiles with two
//     workgroups per CU for the mid-sized ones;
//   * K steps of 64 bytes through NST LDS stages (gemm_direct_body): the smaller tiles, up to four workgroups per
//     CU, the few-rows weight stream (NST = 8 / 16) and the convolution whose activation operand is gathered from
//     the image.
// Any K that is a multiple of 16: the weights are zero padded, so an activation chunk past K only has to be a valid
// read (it re-reads the row's last chunk).  LDS rows are XOR-swizzled in units of 16 bytes so that the 16-byte
// fragment reads of a wave are bank-conflict free.
#include "common.h"
#include "quant_math.h"

#include <stdlib.h>

#include <type_traits>

namespace mi {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

enum { EPI_REQUANT = 0, EPI_DEQUANT = 1 };

struct GemmArgs {
  const int8_t *a;
  int64_t lda;
  int m;
  int k;  // bytes of K that may be read from A (multiple of 16)
  const int8_t *w;
  int ldw;    // weight row stride in bytes
  int k_pad;  // contraction extent of the packed weights (zero filled past K)
  int n;
  int tiles_m, tiles_n;
  void *c;
  int64_t ldc;
  int diag_same_panel;  // timing what-if (wrong results): every tile fetches the operands of tile (0, 0), see diag_same_panel()
};

// Asynchronous 16-byte-per-lane copy global -> LDS: lane L's 16 bytes land at lds_wave_base + 16 * L;
// lds_wave_base must be wave-uniform.  Completion is tracked by vmcnt, in issue order.
__device__ __forceinline__ void async_copy16(const void *global_src, void *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)global_src,
                                   (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

// Hardware deals consecutive workgroup ids round-robin over the 8 XCDs (each with its own L2), so ids that share an
// XCD are mapped to a compact block of tiles, 4 tiles tall: the CUs of one XCD then share operand panels in L2.
__device__ __forceinline__ void tile_coords(const GemmArgs &g, int *tile_m, int *tile_n) {
  int id = blockIdx.x;
  const int nb = gridDim.x, per = nb >> 3;
  if (id < per * 8) id = (id & 7) * per + (id >> 3);
  constexpr int G = 4;
  const int width = G * g.tiles_n;
  const int group = id / width, first = group * G;
  const int gsize = min(g.tiles_m - first, G);
  *tile_m = first + (id % width) % gsize;
  *tile_n = (id % width) / gsize;
}

// clamp to [lo, hi] in one instruction (valid for lo <= hi)
__device__ __forceinline__ int med3_i32(int x, int lo, int hi) {
  int y;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(y) : "v"(x), "v"(lo), "v"(hi));
  return y;
}

__device__ __forceinline__ uint32_t pack4(int y0, int y1, int y2, int y3) {
  // low bytes of four ints -> one dword (v_perm_b32 x3)
  const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)y1, (uint32_t)y0, 0x0c0c0400u);
  const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)y3, (uint32_t)y2, 0x0c0c0400u);
  return __builtin_amdgcn_perm(p23, p01, 0x05040100u);
}

// ---- epilogue.  acc[i][j][4*q + e] is output channel n_w + 32*i + 8*q + 4*h + e of output row m_w + 32*j + r.
//      C rows are written with 4-byte (int8) / 16-byte (fp32) stores; the host guarantees n % 4 == 0, ldc % 4 == 0
//      and an aligned base (it routes other shapes through a padded scratch output). ----
//      Per-channel parameters are read from LDS (array p of kEpiArrays x TILE_N ints, filled by EpiParams below):
//      global loads here would share the vmcnt counter with the output stores and serialise on them. ----
constexpr int kEpiArrays = 6;
constexpr int kDeqStageRowBytes = 144;  // fp32 output staging: 32 columns (128 B) + 16 B so that rows shift banks
// bytes of the wave-private output staging tile behind the parameter arrays
template <int EPI, int TM>
constexpr int epi_stage_bytes() { return EPI == EPI_REQUANT ? 16384 : TM * 32 * kDeqStageRowBytes; }

// The workgroup's per-channel epilogue parameters: thread t holds channel n0 + t of each array (fetched at kernel
// start, so the latency is hidden by the main loop) and drops them into LDS once the main loop is done.
template <int TILE_N, int EPI, bool FAST>
struct EpiParams {
  int v[kEpiArrays];
  __device__ __forceinline__ void fetch(const RequantParams &rq, const DequantParams &dq, int n0, int tid) {
#pragma unroll
    for (int a = 0; a < kEpiArrays; ++a) v[a] = 0;
    if (tid < TILE_N) {
      const int n = n0 + tid;  // arrays are padded to a multiple of 256 channels
      if (EPI == EPI_REQUANT && FAST) {
        v[0] = (int)rq.mult2[n];
        v[1] = (int)rq.c2lo[n];  // arrays 1 and 2 are interleaved in LDS: {lo, hi} of channel t at 2 * t
        v[2] = (int)rq.c2hi[n];
        v[3] = rq.pre[n];
        v[4] = rq.rshift[n];
        v[5] = rq.zw[n];
      } else if (EPI == EPI_REQUANT) {
        v[0] = rq.mult[n];
        v[1] = rq.bias2[n];
        v[2] = rq.rshift[n];
        v[3] = rq.zw[n];
        v[4] = rq.lshift[n];
      } else {
        v[0] = __float_as_int(dq.wscale[n]);
        v[1] = dq.wsum[n];
        v[2] = dq.bias != nullptr ? __float_as_int(dq.bias[n]) : 0;
      }
    }
  }
  // call after a barrier that follows the last LDS read of the main loop; ends with a barrier
  __device__ __forceinline__ void to_lds(int *p, int tid) const {
    if (tid < TILE_N) {
#pragma unroll
      for (int a = 0; a < kEpiArrays; ++a) {
        if (EPI == EPI_REQUANT && FAST && (a == 1 || a == 2)) {
          p[TILE_N + 2 * tid + (a - 1)] = v[a];
        } else {
          p[a * TILE_N + tid] = v[a];
        }
      }
    }
    __syncthreads();
  }
};

// What the fp32 epilogue needs of the input's quantisation.  With DynamicQuant upstream the values live in device
// memory; they are fetched before the main loop, which hides a dependent load of a microsecond that would otherwise
// sit between the last MFMA and the first store of every tile.
template <int TM>
struct DeqInput {
  float sx;
  int32_t zx;
  float sxr[TM];  // per_row: the scale of the rows this lane holds
  __device__ __forceinline__ void fetch(const DequantParams &dq, int m_w, int r, int m_total) {
    sx = dq.sx;
    zx = dq.zx;
    if (dq.qp_dev != nullptr) {
      sx = dq.qp_dev->scale_f;
      zx = dq.qp_dev->zero_point;
    }
    // input_per_channel_: one input scale per row (NN/int8/dynamic_matmul_int8.c:126-128)
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      int m = m_w + j * 32 + r;
      m = m < m_total ? m : m_total - 1;
      sxr[j] = dq.per_row ? dq.qp_dev[m].scale_f : sx;
    }
  }
};

// ACC0: the value the accumulators started from (see kAccBias); it leaves through the per-channel constants, so it
// costs nothing here.
template <int TILE_N, int TN, int TM, int EPI, bool HAS_ZW, bool FAST, uint32_t ACC0 = 0>
__device__ __forceinline__ void gemm_epilogue(v16i (&acc)[TN][TM], int (&rowsum)[TM], const GemmArgs &g,
                                              const RequantParams &rq, const DequantParams &dq,
                                              const DeqInput<TM> din, const int *p, char *cstage, char *cstage_wg,
                                              int n_tile, int m_tile, int n_w, int m_w, int r, int h) {
  static_assert(!(EPI == EPI_REQUANT && FAST) || ACC0 == kAccBias, "the host folds kAccBias into c2");
  if (HAS_ZW) {
#pragma unroll
    for (int j = 0; j < TM; ++j) rowsum[j] += __shfl_xor(rowsum[j], 32);
  }
  if (EPI == EPI_REQUANT) {
    int8_t *c = static_cast<int8_t *>(g.c);
    int amin_v = rq.amin, amax_v = rq.amax;
    asm volatile("" : "+v"(amin_v), "+v"(amax_v));  // kept in vector registers, as v_med3 wants them
    // A 128-channel-wide wave tile goes through LDS so that global memory sees whole 128-byte rows: written
    // straight from the accumulator layout, every store instruction would touch 32 rows with 8 bytes each, and the
    // L2 write path then becomes the bottleneck of the whole kernel.  Wave-private staging tile, 128 rows x 128 B:
    // 16-byte chunk c of row R sits at slot c ^ (R & 7), and inside a chunk dword d sits at (d + (R >> 3)) & 3, which
    // makes both the dword writes (32 rows, one column) and the 16-byte row reads bank-conflict free.
    // The output leaves at memory-write speed (all workgroups reach this point together), and a store instruction
    // that finds the write queue full holds up the wave: so the tile is requantised in two halves of 64 rows, and the
    // eight store instructions of the first half are issued one at a time between the pieces of the second.  (Four
    // passes of 32 rows would hide more of the stores, but every pass re-reads the per-channel constants from LDS,
    // and at four passes those reads take longer than the arithmetic.)
    constexpr bool kStageC = (TN == 4 && TM == 4);
    // The 128 x 128 tile (four wave tiles of 64 channels x 64 rows) does the same through ONE staging tile of
    // 128 rows x 128 B shared by the workgroup (same layout), so that its rows, too, leave as whole 128-byte lines:
    // every wave drops its quadrant, the workgroup meets, every wave stores 32 rows.  Straight from the accumulator
    // layout the stores were a quarter to a third of the launch time of mid-sized shapes (4096 x 1024 x 1024: 2.3 of
    // 9.0 us, 3136 x 2048 x 512: 3.3 of 10.0 us).
    constexpr bool kStageWG = (TN == 2 && TM == 2);
    const int wn_id = (n_w - n_tile) / (32 * TN), wm_id = (m_w - m_tile) / (32 * TM);
    const int lane = h * 32 + r;
    const bool vec16 = ((g.ldc & 15) == 0) && ((reinterpret_cast<uintptr_t>(c) & 15) == 0);
    // four outputs (consecutive channels of one row): accumulator registers -> clamped int32
    auto requant4 = [&](const int32_t (&accv)[4], int rsum, v4i mult, v4i c2lo, v4i c2hi, v4i pre, v4i bias, v4i e4,
                        v4i ls, v4i zw, int (&y)[4]) {
      if (FAST) {
        // the host proved that the accumulator register, read as unsigned, stays below 2^31, that c2 is negative and
        // that none of the sums below leaves its type (RequantParams::fast2).  p2 = a * mult2 + c2 as unsigned 64-bit
        // numbers carries out exactly when the true (signed) sum is >= 0, i.e. when x >= 0: the carry is the
        // "+1 unless negative" of the rounding, so pre arrives here as pre - 1.  The four chains are written stage
        // by stage so that no instruction waits for the one before it.
        uint64_t p2[4], carry[4], unused;
        int32_t t[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          uint32_t a = (uint32_t)accv[e];
          if (HAS_ZW) a -= (uint32_t)rsum * (uint32_t)zw[e];
          const uint64_t c2 = ((uint64_t)(uint32_t)c2hi[e] << 32) | (uint32_t)c2lo[e];
          asm("v_mad_u64_u32 %0, %1, %2, %3, %4" : "=&v"(p2[e]), "=s"(carry[e]) : "v"(a), "v"(mult[e]), "v"(c2));
        }
#pragma unroll
        for (int e = 0; e < 4; ++e)
          asm("v_addc_co_u32_e64 %0, %1, %2, %3, %4"
              : "=v"(t[e]), "=s"(unused)
              : "v"((int32_t)(p2[e] >> 32)), "v"(pre[e]), "s"(carry[e]));
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] >>= e4[e];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = med3_i32(t[e], amin_v, amax_v);
        return;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t v = (uint32_t)accv[e];
        if (HAS_ZW) v -= (uint32_t)rsum * (uint32_t)zw[e];
        v += (uint32_t)bias[e];
        int32_t t = rdiv_pot(srdhm((int32_t)(v << ls[e]), mult[e]), e4[e]);
        t = (int32_t)((uint32_t)t + (uint32_t)rq.zo);
        t = t < rq.amax ? t : rq.amax;
        y[e] = t > rq.amin ? t : rq.amin;
      }
    };
    // whole wave tile inside the matrix and 16-byte stores possible: the stores need no bounds checks
    const bool full_tile = kStageWG ? vec16 && m_tile + 64 * TM <= g.m && n_tile + 64 * TN <= g.n
                                    : vec16 && m_w + 32 * TM <= g.m && n_w + 32 * TN <= g.n;
    // The body is compiled twice: for wave tiles that lie wholly inside the matrix with 16-byte stores possible
    // (no bounds checks, no divergent branches around the stores) and for the ragged rest.
    auto body = [&](auto full_c) {
      constexpr bool FULL = decltype(full_c)::value;
      // rows lrow + 8 * t of the staging tile -> global memory (t: 0..15, one store instruction)
      auto store_rows = [&](int t) {
        const int c16 = lane & 7, lrow = lane >> 3;
        const int n = n_w + c16 * 16;
        const int row = lrow + 8 * t;
        const v4i x = *reinterpret_cast<const v4i *>(cstage + row * 128 + ((c16 ^ lrow) << 4));
        v4i o;  // undo the in-chunk rotation: (row >> 3) & 3 == t & 3
        o[0] = x[(0 + t) & 3];
        o[1] = x[(1 + t) & 3];
        o[2] = x[(2 + t) & 3];
        o[3] = x[(3 + t) & 3];
        const int m = m_w + row;
        if (FULL) {
          // (the staged form only runs on outputs of a dozen megabytes and more: streamed past the L2, they leave no
          //  dirty lines for the end-of-kernel write-back, which otherwise adds ~1.5 us before the next kernel starts)
          __builtin_nontemporal_store(o, reinterpret_cast<v4i *>(c + (int64_t)m * g.ldc + n));
        } else if (m < g.m && n < g.n) {
          int8_t *dst = c + (int64_t)m * g.ldc + n;
          if (vec16 && n + 16 <= g.n) {
            *reinterpret_cast<v4i *>(dst) = o;
          } else {
  #pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + 4 * e < g.n) *reinterpret_cast<int *>(dst + 4 * e) = o[e];
          }
        }
      };
      // the workgroup-shared form: wave w stores rows 32 w .. 32 w + 31 of the tile, 8 per instruction
      auto store_rows_wg = [&](int tt) {
        const int c16 = lane & 7, lrow = lane >> 3;
        const int n = n_tile + c16 * 16;
        const int row = lrow + 8 * (4 * (wm_id * 2 + wn_id) + tt);
        const v4i x = *reinterpret_cast<const v4i *>(cstage_wg + row * 128 + ((c16 ^ lrow) << 4));
        v4i o;  // undo the in-chunk rotation: (row >> 3) & 3 == tt
        o[0] = x[(0 + tt) & 3];
        o[1] = x[(1 + tt) & 3];
        o[2] = x[(2 + tt) & 3];
        o[3] = x[(3 + tt) & 3];
        const int m = m_tile + row;
        if (FULL) {
          *reinterpret_cast<v4i *>(c + (int64_t)m * g.ldc + n) = o;
        } else if (m < g.m && n < g.n) {
          int8_t *dst = c + (int64_t)m * g.ldc + n;
          if (vec16 && n + 16 <= g.n) {
            *reinterpret_cast<v4i *>(dst) = o;
          } else {
  #pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + 4 * e < g.n) *reinterpret_cast<int *>(dst + 4 * e) = o[e];
          }
        }
      };
      constexpr int kPhases = kStageC ? 2 : 1, kJ = TM / kPhases;  // row blocks per pass over the channels
      // where this lane's dword of piece (i, q) goes in its staging row (see the layout above)
      int stage_off[(kStageC || kStageWG) ? TN * 4 : 1];
      if (kStageWG) {
  #pragma unroll
        for (int i = 0; i < TN; ++i)
  #pragma unroll
          for (int q = 0; q < 4; ++q)
            stage_off[i * 4 + q] = (wm_id * 32 * TM + r) * 128 + (((wn_id * 4 + 2 * i + (q >> 1)) ^ (r & 7)) << 4) +
                                   (((2 * q + h + (r >> 3)) & 3) << 2);
      }
      if (kStageC) {
  #pragma unroll
        for (int i = 0; i < TN; ++i)
  #pragma unroll
          for (int q = 0; q < 4; ++q)
            stage_off[i * 4 + q] = r * 128 + (((2 * i + (q >> 1)) ^ (r & 7)) << 4) + (((2 * q + h + (r >> 3)) & 3) << 2);
      }
      // per-channel constants of one piece (4 channels); the next piece's are requested before this piece's
      // arithmetic starts, so that the LDS latency is not paid once per piece
      struct Piece {
        v4i mult4, bias4, e4, zw4, ls4, pre4, c01, c23;
      };
      auto load_piece = [&](int blk) {
        Piece pc;
        const int i = (blk >> 2) % TN, q = blk & 3;
        int nb = n_w + i * 32 + q * 8 + h * 4;
        const int *pl = p + (nb - n_tile);
        pc.mult4 = *reinterpret_cast<const v4i *>(pl);
        pc.bias4 = pc.zw4 = pc.ls4 = pc.pre4 = pc.c01 = pc.c23 = v4i{0, 0, 0, 0};
        if (FAST) {
          pc.c01 = *reinterpret_cast<const v4i *>(p + TILE_N + 2 * (nb - n_tile));  // {lo, hi} x 2
          pc.c23 = *reinterpret_cast<const v4i *>(p + TILE_N + 2 * (nb - n_tile) + 4);
          pc.pre4 = *reinterpret_cast<const v4i *>(pl + 3 * TILE_N);
          pc.e4 = *reinterpret_cast<const v4i *>(pl + 4 * TILE_N);
          if (HAS_ZW) pc.zw4 = *reinterpret_cast<const v4i *>(pl + 5 * TILE_N);
        } else {
          pc.bias4 = *reinterpret_cast<const v4i *>(pl + TILE_N);
          pc.e4 = *reinterpret_cast<const v4i *>(pl + 2 * TILE_N);
          if (HAS_ZW) pc.zw4 = *reinterpret_cast<const v4i *>(pl + 3 * TILE_N);
          pc.ls4 = *reinterpret_cast<const v4i *>(pl + 4 * TILE_N);
  #pragma unroll
          for (int e = 0; e < 4; ++e) pc.bias4[e] = (int32_t)((uint32_t)pc.bias4[e] - ACC0);
        }
        return pc;
      };
      Piece next = load_piece(0);
  #pragma unroll
      for (int ph = 0; ph < kPhases; ++ph) {
  #pragma unroll
        for (int i = 0; i < TN; ++i) {
  #pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int nb = n_w + i * 32 + q * 8 + h * 4;
            const Piece pc = next;
            next = load_piece(i * 4 + q + 1);  // (wraps to piece 0 for the next pass; the arrays are padded)
            // (the staged form computes every channel of the padded tile and lets the stores check the bounds)
            if (!kStageC && !kStageWG && nb >= g.n) continue;
            const v4i c2lo4 = v4i{pc.c01[0], pc.c01[2], pc.c23[0], pc.c23[2]};
            const v4i c2hi4 = v4i{pc.c01[1], pc.c01[3], pc.c23[1], pc.c23[3]};
  #pragma unroll
            for (int jj = 0; jj < kJ; ++jj) {
              const int j = ph * kJ + jj;
              int y[4];
              const int32_t a4[4] = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
              requant4(a4, rowsum[j], pc.mult4, c2lo4, c2hi4, pc.pre4, pc.bias4, pc.e4, pc.ls4, pc.zw4, y);
              const uint32_t packed = pack4(y[0], y[1], y[2], y[3]);
              if (kStageC) {
                *reinterpret_cast<uint32_t *>(cstage + j * 32 * 128 + stage_off[i * 4 + q]) = packed;
              } else if (kStageWG) {
                *reinterpret_cast<uint32_t *>(cstage_wg + j * 32 * 128 + stage_off[i * 4 + q]) = packed;
              } else {
                const int m = m_w + j * 32 + r;
                if (m < g.m) *reinterpret_cast<uint32_t *>(c + (int64_t)m * g.ldc + nb) = packed;
              }
            }
            if (kStageC && ph == 1 && (q & 1)) {  // the first half's eight store instructions, one per two pieces
              __builtin_amdgcn_sched_barrier(0);
              store_rows(i * 2 + (q >> 1));
              __builtin_amdgcn_sched_barrier(0);
            }
          }
        }
      }
      if (kStageC) {
  #pragma unroll
        for (int t = 8; t < 16; ++t) store_rows(t);
      }
      if (kStageWG) {
        __syncthreads();
  #pragma unroll
        for (int tt = 0; tt < 4; ++tt) store_rows_wg(tt);
      }
    };
    if (full_tile) {
      body(std::true_type());
    } else {
      body(std::false_type());
    }
  } else {
    float *c = static_cast<float *>(g.c);
    const int32_t zx = din.zx;
    const uint32_t kzz = (uint32_t)dq.deep * (uint32_t)zx * (uint32_t)dq.zw0;
    // As for the int8 output, the accumulator layout (a lane holds 4 consecutive columns of 32 different rows) is
    // turned into whole 128-byte row segments before it meets global memory: per 32-column block the wave's
    // TM x 32 rows go through a wave-private LDS tile (row stride 144 bytes: the 16-byte writes of 8 consecutive
    // rows and the 16-byte reads along a row are both bank-conflict free) and leave as 8 rows x 128 B per store.
    constexpr int kRowB = kDeqStageRowBytes;
    const int lane = h * 32 + r;
    const int lr = lane >> 3, lc = lane & 7;
    const bool has_bias = dq.bias != nullptr;
    // The body exists three times, chosen once per tile instead of with branches around every output: full tile
    // without activation and with one input scale (no bounds compares, no clamps, the scale product hoisted), full
    // tile in general, ragged tile in general.
    // The general bodies clamp between bounds that are infinite where the reference makes no comparison: (-inf > d)
    // and (inf < d) are false for every d, NaN included, so no activation, ReLU and ReLU6 share one form.
    const bool with_act = dq.act == MI_ACT_RELU || dq.act == MI_ACT_RELU6;
    const float act_lo = with_act ? 0.0f : -__builtin_inff();
    const float act_hi = dq.act == MI_ACT_RELU6 ? 6.0f : __builtin_inff();
    auto body = [&](auto full_c, auto act_c, auto rows_c) {
      constexpr bool FULL = decltype(full_c)::value, ACT = decltype(act_c)::value, PER_ROW = decltype(rows_c)::value;
#pragma unroll
      for (int i = 0; i < TN; ++i) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int nb = n_w + i * 32 + q * 8 + h * 4;
          const int *pl = p + (nb - n_tile);
          const v4f ws4 = *reinterpret_cast<const v4f *>(pl);
          const v4i wsum4 = *reinterpret_cast<const v4i *>(pl + TILE_N);
          const v4f b4 = *reinterpret_cast<const v4f *>(pl + 2 * TILE_N);
          uint32_t corr[4];
          float s4[4];  // one input scale for the whole tensor: the scale product is the same for every row
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            corr[e] = kzz - (uint32_t)zx * (uint32_t)wsum4[e] - ACC0;
            s4[e] = __fmul_rn(din.sx, ws4[e]);
          }
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            v4f o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              uint32_t v = (uint32_t)acc[i][j][q * 4 + e] + corr[e];
              if (HAS_ZW) v -= (uint32_t)dq.zw0 * (uint32_t)rowsum[j];
              float d = __fmul_rn(PER_ROW ? __fmul_rn(din.sxr[j], ws4[e]) : s4[e], (float)(int32_t)v);
              if (has_bias) d = __fadd_rn(d, b4[e]);
              if (ACT) {
                d = (act_lo > d) ? act_lo : d;
                d = (act_hi < d) ? act_hi : d;
              }
              o[e] = d;
            }
            *reinterpret_cast<v4f *>(cstage + (j * 32 + r) * kRowB + (q * 8 + h * 4) * 4) = o;
          }
        }
        const int n = n_w + i * 32 + lc * 4;
#pragma unroll
        for (int t = 0; t < TM * 4; ++t) {
          const int row = t * 8 + lr;
          const v4f v = *reinterpret_cast<const v4f *>(cstage + row * kRowB + lc * 16);
          const int m = m_w + row;
          if (FULL || (m < g.m && n < g.n)) {
            v4f *dst = reinterpret_cast<v4f *>(c + (int64_t)m * g.ldc + n);
            if (FAST) {  // in this epilogue the parameter selects non-temporal stores (see stream_out_hint)
              __builtin_nontemporal_store(v, dst);
            } else {
              *dst = v;
            }
          }
        }
      }
    };
    const bool full_tile = m_w + 32 * TM <= g.m && n_w + 32 * TN <= g.n;
    // (the common case, a full tile of a MatMul without activation and with one input scale, has a body of its own;
    //  per-row scales and activations share the general one)
    if (full_tile && !with_act && !dq.per_row) {
      body(std::true_type(), std::false_type(), std::false_type());
    } else if (full_tile) {
      body(std::true_type(), std::true_type(), std::true_type());
    } else {
      body(std::false_type(), std::true_type(), std::true_type());
    }
  }
}

template <int TN, int TM>
struct Frag {
  v4i w[TN], a[TM];
};

template <int TN, int TM, bool HAS_ZW>
__device__ __forceinline__ void mma_frag(v16i (&acc)[TN][TM], int (&rowsum)[TM], const Frag<TN, TM> &f, int ones) {
  // ones: 0x01010101, or 0 when this lane's 16 activation bytes lie past K (they are then a re-read of valid
  // bytes, harmless for the products because the weights are zero there, but they must not enter the row sums)
  if (HAS_ZW) {
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      int t = rowsum[j];
      t = __builtin_amdgcn_sdot4(f.a[j].x, ones, t, false);
      t = __builtin_amdgcn_sdot4(f.a[j].y, ones, t, false);
      t = __builtin_amdgcn_sdot4(f.a[j].z, ones, t, false);
      t = __builtin_amdgcn_sdot4(f.a[j].w, ones, t, false);
      rowsum[j] = t;
    }
  }
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[i], f.a[j], acc[i][j], 0, 0, 0);
}

// Instruction-order hints for one K sub-step: spread the LDS operand reads between the MFMAs instead of issuing them
// in one burst, so that the matrix pipe always has the next MFMA queued.
template <int TN, int TM>
__device__ __forceinline__ void hint_interleave_reads() {
  // one read after each of the first MFMAs: the reads are all issued early in the sub-step, so their data has the
  // remaining MFMAs' time to arrive before the next sub-step needs it
  constexpr int kReads = TN + TM, kMfma = TN * TM;
  if constexpr (kMfma >= kReads) {
#pragma unroll
    for (int i = 0; i < kReads; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
    }
  } else {
#pragma unroll
    for (int i = 0; i < kMfma; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, kReads / kMfma, 0);
    }
  }
}

// =====================================================================================================================
// direct main loop: NST LDS stages x 64 bytes of K, asynchronous global -> LDS loads NST - 1 tiles ahead.
// NST = 4 for the compute-bound shapes (3 for short K, where a third workgroup per CU is worth more than depth); NST = 16 with 64 x 64 tiles for a few (<= 64) activation rows, where the
// kernel is a weight stream and what counts is the number of bytes in flight per CU.
// OCC = workgroups the register allocation leaves room for on one CU (waves per SIMD): 1 for the 256 x 256 tile, which
// needs the whole register file, 2 for the 128 x 128 tile.
// =====================================================================================================================
// CONV: the activation operand is not a matrix in memory but the im2col view of an NHWC image (in_c % 16 == 0): row m
// is output pixel m, and the 16-byte chunk at K offset k is 16 channels of tap k / in_c, fetched straight from the
// image, or from 16 bytes of the fill value when the tap lies outside the image (conv_int8.c:758-807,877).
struct ConvGather {
  int in_h, in_w, in_c, out_w, out_hw;
  int kernel_w, stride_h, stride_w, dil_h, dil_w, pad_u, pad_l;
  uint32_t magic_ic, magic_kw;  // ceil(2^32 / in_c), ceil(2^32 / kernel_w): exact quotients for dividends < 2^16
  const int8_t *fill16;
};

template <int TILE_N, int TILE_M, int EPI, bool HAS_ZW, bool FAST, int NST, bool CONV>
__device__ __forceinline__ void gemm_direct_body(const GemmArgs &g, const RequantParams &rq, const DequantParams &dq,
                                                 const ConvGather &cv) {
  constexpr int BKD = 64, PD = NST - 1;  // PD: prefetch distance in K steps
  static_assert(NST >= 3, "the loop keeps NST - 1 >= 2 tiles in flight");
  auto wrap = [](int x) { return x >= NST ? x - NST : x; };  // stage index after an increment of at most NST
  constexpr int WN = TILE_N / 2, WM = TILE_M / 2, TN = WN / 32, TM = WM / 32;
  constexpr int STAGE = (TILE_N + TILE_M) * BKD;
  constexpr int WPW = TILE_N / 16 / 4, APW = TILE_M / 16 / 4, LPW = WPW + APW;  // 1 KiB blocks per wave and tile
  static_assert(WPW >= 1 && APW >= 1, "tile too small");
  static_assert(EPI != EPI_REQUANT || TN != 2 || TM != 2 || NST * STAGE >= kEpiArrays * TILE_N * 4 + 16384,
                "the workgroup's output staging tile must fit the main loop's LDS");
  static_assert(EPI == EPI_REQUANT ? (TN != 4 || TM != 4 || NST * STAGE >= kEpiArrays * TILE_N * 4 + 4 * 16384)
                                   : NST * STAGE >= kEpiArrays * TILE_N * 4 + 4 * epi_stage_bytes<EPI, TM>(),
                "the epilogue staging must fit the main loop's LDS");
  __shared__ __attribute__((aligned(1024))) char lds[NST * STAGE];

  int tile_m, tile_n;
  tile_coords(g, &tile_m, &tile_n);
  const int m0 = tile_m * TILE_M, n0 = tile_n * TILE_N;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int r = lane & 31, h = lane >> 5;
  const int ktiles = (g.k + BKD - 1) / BKD;  // the zero padding of the weights past K needs no MFMAs
  const int kchunks = g.k >> 4;
  EpiParams<TILE_N, EPI, FAST> epi;
  epi.fetch(rq, dq, n0, tid);
  DeqInput<TM> din;
  if (EPI == EPI_DEQUANT) din.fetch(dq, m0 + wm * WM, r, g.m);

  // loader: a 1 KiB block holds 16 rows x 64 B.  Lane L fills slot (L & 3) of row (L >> 2) of its block, i.e. it
  // fetches logical chunk (L & 3) ^ swizzle(row), swizzle(row) = (row >> 1) & 3.
  const int drow = lane >> 2;
  const int dchunk = (lane & 3) ^ ((lane >> 3) & 3);
  const int8_t *wsrc = g.w + (int64_t)(n0 + wave * WPW * 16 + drow) * g.ldw + dchunk * 16;
  const int8_t *asrc[APW];
  int ih0[CONV ? APW : 1], iw0[CONV ? APW : 1];
#pragma unroll
  for (int i = 0; i < APW; ++i) {
    int m = m0 + (wave * APW + i) * 16 + drow;
    m = m < g.m ? m : g.m - 1;
    if (CONV) {
      const int b = m / cv.out_hw, rem = m - b * cv.out_hw;
      const int oh = rem / cv.out_w, ow = rem - oh * cv.out_w;
      ih0[i] = oh * cv.stride_h - cv.pad_u;
      iw0[i] = ow * cv.stride_w - cv.pad_l;
      // address of (ih0, iw0, channel 0); only dereferenced for taps inside the image
      asrc[i] = g.a + (((int64_t)b * cv.in_h + ih0[i]) * cv.in_w + iw0[i]) * cv.in_c;
    } else {
      asrc[i] = g.a + (int64_t)m * g.lda;
    }
  }
  // A has exactly K valid bytes per row (the weights are zero padded, A is the caller's): a 16-byte chunk past K is
  // fetched from the row's last chunk instead
  const int a_last = (kchunks - 1) * 16;
  auto dma_tile = [&](int stage, int kt) {
    char *sw = lds + stage * STAGE + wave * WPW * 1024;
    char *sa = lds + stage * STAGE + TILE_N * BKD + wave * APW * 1024;
#pragma unroll
    for (int i = 0; i < WPW; ++i) async_copy16(wsrc + (int64_t)i * 16 * g.ldw + kt * BKD, sw + i * 1024);
    int koff = kt * BKD + dchunk * 16;
    if (CONV) {
      const uint32_t tap = __umulhi((uint32_t)koff, cv.magic_ic);
      const int ic = koff - (int)tap * cv.in_c;
      const uint32_t kh = cv.kernel_w == 1 ? tap : __umulhi(tap, cv.magic_kw);
      const int dh = (int)kh * cv.dil_h, dw = ((int)tap - (int)kh * cv.kernel_w) * cv.dil_w;
      const int tap_off = (dh * cv.in_w + dw) * cv.in_c + ic;
      const bool in_k = koff < g.k;  // past K the weights are zero: any 16 readable bytes will do
#pragma unroll
      for (int i = 0; i < APW; ++i) {
        const int ih = ih0[i] + dh, iw = iw0[i] + dw;
        const bool inside = in_k && (unsigned)ih < (unsigned)cv.in_h && (unsigned)iw < (unsigned)cv.in_w;
        async_copy16(inside ? asrc[i] + tap_off : cv.fill16, sa + i * 1024);
      }
      return;
    }
    koff = koff < a_last ? koff : a_last;
#pragma unroll
    for (int i = 0; i < APW; ++i) async_copy16(asrc[i] + koff, sa + i * 1024);
  };

  v16i acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = (int)kAccBias;  // see gemm_kblock_kernel
  int rowsum[TM];
#pragma unroll
  for (int j = 0; j < TM; ++j) rowsum[j] = 0;

  // operand fragments: this lane's rows are r + multiples of 32, so its swizzle is a lane constant
  const int frag_swz = (r >> 1) & 3;
  const int w_off = (wn * WN + r) * BKD, a_off = TILE_N * BKD + (wm * WM + r) * BKD;
  Frag<TN, TM> f0, f1;
  auto read_frag = [&](Frag<TN, TM> &f, int stage, int s) {
    const char *base = lds + stage * STAGE + (((2 * s + h) ^ frag_swz) << 4);
#pragma unroll
    for (int i = 0; i < TN; ++i) f.w[i] = *reinterpret_cast<const v4i *>(base + w_off + i * 32 * BKD);
#pragma unroll
    for (int j = 0; j < TM; ++j) f.a[j] = *reinterpret_cast<const v4i *>(base + a_off + j * 32 * BKD);
  };
  // One 64-byte K step on LDS stage `st` (tile kt).  On entry f0 holds sub-step 0 of this stage.
  //   sub-step 0 : MFMAs on f0 while f1 <- sub-step 1 of this stage
  //   barrier    : first wait until at most (PD - 2) * LPW of this wave's loads are outstanding (loads complete in
  //                order, so that is "tile kt+1 has landed, later tiles may still be in flight"), then meet the other
  //                waves: now tile kt+1 is complete in LDS and nobody reads stage st-1 (tile kt-1) any more
  //   sub-step 1 : refill that stage with tile kt+PD, f0 <- sub-step 0 of tile kt+1, MFMAs on f1
  // With more than four stages the loads past the end of K re-fetch the last tile into a stage nobody reads again,
  // which keeps the outstanding-load count the same in every step; with up to four the last steps are separate
  // bodies without loads (see below).
  auto step = [&](int kt, int st) {
    read_frag(f1, st, 1);
    mma_frag<TN, TM, HAS_ZW>(acc, rowsum, f0, (kt * 4 + h < kchunks) ? 0x01010101 : 0);
    hint_interleave_reads<TN, TM>();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((PD - 2) * LPW) : "memory");
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    const int nxt = kt + PD < ktiles ? kt + PD : ktiles - 1;
    read_frag(f0, wrap(st + 1), 0);
    dma_tile(wrap(st + PD), nxt);
    mma_frag<TN, TM, HAS_ZW>(acc, rowsum, f1, (kt * 4 + 2 + h < kchunks) ? 0x01010101 : 0);
    {
      // operand reads first (the next sub-step waits for them), the loads of tile kt+3 behind them (they have
      // almost three steps to land)
      constexpr int kMfma = TN * TM, kReads = TN + TM;
      if constexpr (kMfma >= kReads + LPW) {
#pragma unroll
        for (int i = 0; i < kReads; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
        }
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global -> LDS load issue
        }
      } else {
#pragma unroll
        for (int i = 0; i < kMfma; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, (kReads + kMfma - 1) / kMfma, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, (LPW + kMfma - 1) / kMfma, 0);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
#pragma unroll
  for (int t = 0; t < PD; ++t) dma_tile(t, t < ktiles ? t : ktiles - 1);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((PD - 1) * LPW) : "memory");
  read_frag(f0, 0, 0);
  if constexpr (NST <= 4) {
    // The last PD steps have bodies of their own that load nothing: with a dozen K steps, as in the K = 768 shapes,
    // re-fetching the last tile PD times is a fifth of the operand traffic.  REM = tiles after this one; the tiles
    // still in flight at its wait are kt+2 .. the last one.
    auto tail_step = [&](int kt, int st, auto rem_c) {
      constexpr int REM = decltype(rem_c)::value;
      read_frag(f1, st, 1);
      mma_frag<TN, TM, HAS_ZW>(acc, rowsum, f0, (kt * 4 + h < kchunks) ? 0x01010101 : 0);
      hint_interleave_reads<TN, TM>();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (REM >= 1) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((REM - 1) * LPW) : "memory");
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        read_frag(f0, wrap(st + 1), 0);
      }
      mma_frag<TN, TM, HAS_ZW>(acc, rowsum, f1, (kt * 4 + 2 + h < kchunks) ? 0x01010101 : 0);
      hint_interleave_reads<TN, TM>();
      __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0, st = 0;
    for (; kt + PD < ktiles; ++kt, st = wrap(st + 1)) step(kt, st);
    if constexpr (PD >= 3) {
      if (ktiles - 1 - kt == 2) {
        tail_step(kt, st, std::integral_constant<int, 2>());
        ++kt;
        st = wrap(st + 1);
      }
    }
    if (ktiles - 1 - kt == 1) {
      tail_step(kt, st, std::integral_constant<int, 1>());
      ++kt;
      st = wrap(st + 1);
    }
    tail_step(kt, st, std::integral_constant<int, 0>());
  } else {
    for (int kt = 0, st = 0; kt < ktiles; ++kt, st = wrap(st + 1)) step(kt, st);
  }
  // (also: every load must have landed before the LDS is reused below or handed to another workgroup)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  epi.to_lds(reinterpret_cast<int *>(lds), tid);
  gemm_epilogue<TILE_N, TN, TM, EPI, HAS_ZW, FAST, kAccBias>(
      acc, rowsum, g, rq, dq, din, reinterpret_cast<const int *>(lds),
      lds + kEpiArrays * TILE_N * 4 + wave * epi_stage_bytes<EPI, TM>(), lds + kEpiArrays * TILE_N * 4, n0, m0,
      n0 + wn * WN, m0 + wm * WM, r, h);
}

template <int TILE_N, int TILE_M, int EPI, bool HAS_ZW, bool FAST, int NST, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void gemm_direct_kernel(GemmArgs g, RequantParams rq, DequantParams dq) {
  gemm_direct_body<TILE_N, TILE_M, EPI, HAS_ZW, FAST, NST, false>(g, rq, dq, ConvGather{});
}

// The same GEMM with the activation operand gathered from an NHWC image (no im2col buffer).
template <int TILE_N, int TILE_M, bool HAS_ZW, bool FAST, int NST, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void gemm_conv_kernel(GemmArgs g, ConvGather cv, RequantParams rq) {
  gemm_direct_body<TILE_N, TILE_M, EPI_REQUANT, HAS_ZW, FAST, NST, true>(g, rq, DequantParams{}, cv);
}

// =====================================================================================================================
// K-block main loop for the 256 x 256 tile (one workgroup per CU, the whole register file).
//
// What the compute-bound GEMM pays for is operand delivery: the L2 -> L1 path moves whole 128-byte lines, so a loader
// that asks for 64 bytes of a row per K step has every line sent twice, one K step apart.  Here K advances in blocks of 128 bytes
// -- whole cache lines -- so that each line leaves the L2 once: one wave instruction fetches 8 rows x 128 bytes.
// LDS holds three slots for W and two for A (slot = 256 rows x 128 B = 32 KiB; all 160 KiB of the CU).  The path from
// the L1 into LDS moves 64 bytes per clock and CU: four waves issuing eight 1 KiB loads each within one quarter of a
// block saturate it, and a wave whose load does not fit the queue cannot issue its next MFMA either.  So every quarter
// issues four loads per wave, which takes a load window of a whole block per operand, hence the third W slot.  A loop
// iteration is one K block = four 32-byte MFMA sub-steps (quarters) on double-buffered fragments:
//   Q1  MFMAs on chunks 0-1 | reads chunks 2-3 | loads the second half of A block b+1
//   Q2  MFMAs on chunks 2-3 | reads chunks 4-5 | loads the first half of W block b+2 (into block b-1's slot)
//   Q3  MFMAs on chunks 4-5 | reads chunks 6-7 | loads the second half of W block b+2, then waits until all but
//       these eight W loads have landed (loads complete in order) and meets the other waves: block b+1 is complete
//       in LDS and nobody reads block b any more
//   Q4  MFMAs on chunks 6-7 | reads chunks 0-1 of block b+1 | loads the first half of A block b+2 into block b's slot
// One barrier per 128 bytes of K.  In a slot, 16-byte chunk c of row R sits at position c ^ ((R >> 1) & 7): the LDS
// has 64 banks (256 bytes per clock), so 16 consecutive rows of one logical chunk -- what 16 lanes of a fragment
// read ask for -- must land on 16 different 16-byte positions of a 256-byte period, and two rows of 128 bytes make
// one period.
//
// kAccBias: the accumulators start from this constant instead of 0 and the epilogue's per-channel constants take it
// out again (exact: wrap-around arithmetic).  Partial sums of signed products hover around zero, where every sign
// change flips all upper bits of the 32-bit accumulator; from an alternating bit pattern a sum that crosses it
// flips at most the bits up to the next 0/1 boundary.  The matrix pipe alone, on operands drawn like this
// benchmark's, sustains 7-9 % more (power-limited shader clock) with it.  For the same reason consecutive MFMAs
// share one operand (serpentine order over the 4 x 4 sub-tiles): +5 %.
// =====================================================================================================================
// T: the wave's sub-tile is T x T MFMA tiles, the workgroup's tile 64 T x 64 T.  T = 4 is the 256 x 256 tile described
// above.  T = 2 (128 x 128, slots of 16 KiB, 80 KiB of LDS, a quarter of the registers) lets two workgroups share a
// CU: for shapes with fewer than one 256 x 256 tile per CU, or short K, where one tile's prologue and epilogue have
// to overlap another tile's main loop.  Per quarter a wave then has 4 MFMAs, 4 fragment reads and 2 loads.
// DIAG: timing what-ifs of the main loop (wrong results, see diag_kblock128()): bit 0 = no operand loads after the
// first two K blocks, bit 1 = no wait and no barrier between K blocks.
template <int T, int EPI, bool HAS_ZW, bool FAST, int DIAG = 0>
__device__ __forceinline__ void gemm_kblock_body(const GemmArgs &g, const RequantParams &rq, const DequantParams &dq) {
#if defined(__HIP_DEVICE_COMPILE__)  // the buffer-resource type exists in the device pass only; the host pass needs just the stub
  constexpr int TILE = 64 * T, KB = 128;  // wave tile 32 T x 32 T = T x T MFMA tiles
  constexpr int SLOT = TILE * KB;         // one operand, one K block
  constexpr int WROWS = TILE / 4;         // rows of each operand that a wave loads per block
  constexpr int LPW = WROWS / 8;          // loader instructions per wave, operand and block (8 rows each)
  static_assert(T == 2 || T == 4, "wave tiles of 64 x 64 or 128 x 128");
  static_assert(5 * SLOT >= kEpiArrays * TILE * 4 + 4 * epi_stage_bytes<EPI, T>(), "the epilogue staging must fit");
  __shared__ __attribute__((aligned(1024))) char lds[5 * SLOT];  // W slots 0-2, A slots 0-1

  int tile_m, tile_n;
  tile_coords(g, &tile_m, &tile_n);
  const int m0 = tile_m * TILE, n0 = tile_n * TILE;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 1, wm = wave >> 1;
  const int r = lane & 31, h = lane >> 5;
  const int kblocks = (g.k + KB - 1) / KB;
  const int kchunks = g.k >> 4;
  EpiParams<TILE, EPI, FAST> epi;
  epi.fetch(rq, dq, n0, tid);
  DeqInput<T> din;
  if (EPI == EPI_DEQUANT) din.fetch(dq, m0 + wm * 32 * T, r, g.m);

  // loader: instruction i of a wave fills rows WROWS * wave + 8 * i + (lane >> 3) of a slot; lane L writes position
  // L & 7 of its row, i.e. fetches logical chunk (L & 7) ^ ((row >> 1) & 7).  The loads are buffer loads: the address
  // is descriptor base + per-lane byte offset (a loop constant) + a scalar offset (row group and K block), so
  // issuing one costs scalar instructions only.
  const int drow = lane >> 3;
  const int dchunk = (lane & 7) ^ (drow >> 1);  // for even i; odd i: ^ 4
  const int ld_n0 = g.diag_same_panel ? 0 : n0, ld_m0 = g.diag_same_panel ? 0 : m0;
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<int8_t *>(g.w) + (int64_t)(ld_n0 + wave * WROWS) * g.ldw, (short)0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(g.a) + (int64_t)ld_m0 * g.lda, (short)0, -1, 0x00020000);
  const int w_voff = drow * g.ldw + dchunk * 16;  // ldw is a multiple of 256: odd i is w_voff ^ 64
  int a_voff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    int m = wave * WROWS + 8 * i + drow;
    m = m0 + m < g.m ? m : g.m - 1 - m0;
    a_voff[i] = m * (int)g.lda + ((dchunk ^ ((i & 1) << 2)) << 4);
  }
  // A has exactly K valid bytes per row (the weights are zero padded, A is the caller's): in the last K block a
  // 16-byte chunk past K is fetched from the row's last chunk instead.  The offsets are moved there once, before
  // that block is first requested (in the 256 x 256 form the re-fetches after it ask for the same block).
  const int a_last = (kchunks - 1) * 16 - (kblocks - 1) * KB;  // offset of the last valid chunk in the last block
  auto a_offsets_for_last_block = [&]() {
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int c16 = (dchunk ^ ((i & 1) << 2)) << 4;
      a_voff[i] += (c16 < a_last ? c16 : a_last) - c16;
    }
  };
  auto lds_ptr = [](char *p) { return (__attribute__((address_space(3))) void *)p; };
  // half: 0 = the first half of the wave's loader instructions (the upper half of its rows), 1 = the other half
  auto dma_w = [&](int slot, int kb, int half) {
    if ((DIAG & 1) && kb > 1) return;
    char *dst = lds + slot * SLOT + wave * WROWS * KB;
#pragma unroll
    for (int ii = 0; ii < LPW / 2; ++ii) {
      const int i = half * (LPW / 2) + ii;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, lds_ptr(dst + i * 1024), 16, w_voff ^ ((i & 1) << 6),
                                               8 * i * g.ldw + kb * KB, 0, 0);
    }
  };
  auto dma_a = [&](int slot, int kb, int half) {
    if ((DIAG & 1) && kb > 1) return;
    char *dst = lds + (3 + slot) * SLOT + wave * WROWS * KB;
#pragma unroll
    for (int ii = 0; ii < LPW / 2; ++ii) {
      const int i = half * (LPW / 2) + ii;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, lds_ptr(dst + i * 1024), 16, a_voff[i], kb * KB, 0, 0);
    }
  };

  v16i acc[T][T];
  int rowsum[T];
#pragma unroll
  for (int j = 0; j < T; ++j) rowsum[j] = 0;
  // the accumulator registers are set while the first tiles are on their way (see below)
  auto init_accumulators = [&]() {
    const int bias = (int)kAccBias;
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
      for (int j = 0; j < T; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e)  // volatile: stays ahead of the wait for the first tiles
          asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(acc[i][j][e]) : "v"(bias));
  };

  const int swz = (r >> 1) & 7;
  const int w_off = (wn * 32 * T + r) * KB, a_off = 3 * SLOT + (wm * 32 * T + r) * KB;
  Frag<T, T> f0, f1;
  auto read_frag = [&](Frag<T, T> &f, int wslot, int aslot, int q) {  // q: 32-byte sub-step inside the block
    const int c = ((2 * q + h) ^ swz) << 4;
    const char *wb = lds + wslot * SLOT + w_off + c, *ab = lds + aslot * SLOT + a_off + c;
#pragma unroll
    for (int i = 0; i < T; ++i) f.w[i] = *reinterpret_cast<const v4i *>(wb + i * 32 * KB);
#pragma unroll
    for (int j = 0; j < T; ++j) f.a[j] = *reinterpret_cast<const v4i *>(ab + j * 32 * KB);
  };
  auto mma = [&](const Frag<T, T> &f, int chunk) {
    if (HAS_ZW) {
      const int ones = chunk < kchunks ? 0x01010101 : 0;
#pragma unroll
      for (int j = 0; j < T; ++j) {
        int t = rowsum[j];
        t = __builtin_amdgcn_sdot4(f.a[j].x, ones, t, false);
        t = __builtin_amdgcn_sdot4(f.a[j].y, ones, t, false);
        t = __builtin_amdgcn_sdot4(f.a[j].z, ones, t, false);
        t = __builtin_amdgcn_sdot4(f.a[j].w, ones, t, false);
        rowsum[j] = t;
      }
    }
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
      for (int jj = 0; jj < T; ++jj) {
        const int j = (i & 1) ? T - 1 - jj : jj;
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.w[i], f.a[j], acc[i][j], 0, 0, 0);
      }
  };
  // T = 4: one LDS read behind each of the first 8 MFMAs of a quarter, then one load behind every other one of the
  // rest.  T = 2: a read behind each of the 4 MFMAs, a load behind every other one.
  auto hints = [&]() {
    if constexpr (T == 4) {
#pragma unroll
      for (int i = 0; i < 2 * T; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
      }
#pragma unroll
      for (int i = 0; i < LPW / 2; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global -> LDS load issue
      }
    } else {
#pragma unroll
      for (int i = 0; i < LPW / 2; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  const int last = kblocks - 1;
  if (kblocks == 1) a_offsets_for_last_block();
  dma_w(0, 0, 0);
  dma_w(0, 0, 1);
  dma_a(0, 0, 0);
  dma_a(0, 0, 1);
  if (kblocks == 2) a_offsets_for_last_block();
  dma_w(1, last < 1 ? last : 1, 0);
  dma_w(1, last < 1 ? last : 1, 1);
  dma_a(1, last < 1 ? last : 1, 0);
  init_accumulators();
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(LPW + LPW / 2) : "memory");  // W(0) and A(0) are in
  read_frag(f0, 0, 0, 0);
  int ws = 0, ws1 = 1, ws2 = 2;  // W slots of blocks b, b+1, b+2
  auto k_block_clamped = [&](int b) {
    const int as = b & 1;
    const int kb1 = b + 1 < last ? b + 1 : last;  // past the end: the last block again, into a slot nobody reads
    const int kb2 = b + 2 < last ? b + 2 : last;
    read_frag(f1, ws, as, 1);
    dma_a(as ^ 1, kb1, 1);
    mma(f0, b * 8 + h);
    hints();
    read_frag(f0, ws, as, 2);
    dma_w(ws2, kb2, 0);
    mma(f1, b * 8 + 2 + h);
    hints();
    read_frag(f1, ws, as, 3);
    dma_w(ws2, kb2, 1);
    mma(f0, b * 8 + 4 + h);
    hints();
    // everything but the eight loads of W block b+2 has landed: that includes all of block b+1
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(LPW) : "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (b + 3 == kblocks) a_offsets_for_last_block();
    read_frag(f0, ws1, as ^ 1, 0);
    dma_a(as, kb2, 0);
    mma(f1, b * 8 + 6 + h);
    hints();
    const int t = ws;
    ws = ws1;
    ws1 = ws2;
    ws2 = t;
  };
  // One K block.  NEXT1 / NEXT2: blocks b + 1 / b + 2 exist.  The last two blocks have their own copies of the body
  // without the loads for blocks that do not exist (with 6 K blocks those would be a third of the operand traffic),
  // and the last one also without the barrier and the read-ahead.
  auto k_block = [&](int b, auto next1_c, auto next2_c) {
    constexpr bool NEXT1 = decltype(next1_c)::value, NEXT2 = decltype(next2_c)::value;
    const int as = b & 1;
    read_frag(f1, ws, as, 1);
    if (NEXT1) dma_a(as ^ 1, b + 1, 1);
    mma(f0, b * 8 + h);
    hints();
    read_frag(f0, ws, as, 2);
    if (NEXT2) dma_w(ws2, b + 2, 0);
    mma(f1, b * 8 + 2 + h);
    hints();
    read_frag(f1, ws, as, 3);
    if (NEXT2) dma_w(ws2, b + 2, 1);
    mma(f0, b * 8 + 4 + h);
    hints();
    if (DIAG & 2) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (NEXT2) {
      // everything but the loads of W block b+2 has landed: that includes all of block b+1
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(LPW) : "memory");
    } else if (NEXT1) {
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // block b+1, the last one, is in
    }
    __builtin_amdgcn_sched_barrier(0);
    if (NEXT2 && b + 3 == kblocks) a_offsets_for_last_block();
    if (NEXT1) read_frag(f0, ws1, as ^ 1, 0);
    if (NEXT2) dma_a(as, b + 2, 0);
    mma(f1, b * 8 + 6 + h);
    hints();
    const int t = ws;
    ws = ws1;
    ws1 = ws2;
    ws2 = t;
  };
  if constexpr (T == 2) {
    for (int b = 0; b + 2 < kblocks; ++b) k_block(b, std::true_type(), std::true_type());
    if (kblocks >= 2) k_block(last - 1, std::true_type(), std::false_type());
    k_block(last, std::false_type(), std::false_type());
  } else {
    // (three copies of the 64-MFMA body push the 256 x 256 tile's register allocation into spilling, and at its
    //  K the two blocks' worth of extra loads are a few per cent: it keeps one body and lets the loads past the
    //  end fetch the last block again, into slots nobody reads)
    for (int b = 0; b < kblocks; ++b) k_block_clamped(b);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every load has landed before the LDS is reused
  __syncthreads();
  epi.to_lds(reinterpret_cast<int *>(lds), tid);
  gemm_epilogue<TILE, T, T, EPI, HAS_ZW, FAST, kAccBias>(acc, rowsum, g, rq, dq, din, reinterpret_cast<const int *>(lds),
                                                         lds + kEpiArrays * TILE * 4 + wave * epi_stage_bytes<EPI, T>(),
                                                         lds + kEpiArrays * TILE * 4, n0, m0, n0 + wn * 32 * T,
                                                         m0 + wm * 32 * T, r, h);
#endif
}

template <int EPI, bool HAS_ZW, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_kblock_kernel(GemmArgs g,
                                                                                                      RequantParams rq,
                                                                                                      DequantParams dq) {
  gemm_kblock_body<4, EPI, HAS_ZW, FAST>(g, rq, dq);
}

// The 128 x 128 form, two workgroups per CU.
template <int EPI, bool HAS_ZW, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_kblock128_kernel(
    GemmArgs g, RequantParams rq, DequantParams dq) {
  gemm_kblock_body<2, EPI, HAS_ZW, FAST>(g, rq, dq);
}

template <int EPI, int DIAG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_kblock128_diag_kernel(
    GemmArgs g, RequantParams rq, DequantParams dq) {
  gemm_kblock_body<2, EPI, false, true, DIAG>(g, rq, dq);
}

// ---- host side -----------------------------------------------------------------------------------------------
// Measurement aid, off unless the environment says MI355X_DIAG_SAME_PANEL=1 when the library is first used: the
// K-block kernels then fetch tile (0, 0)'s operands for every tile, so that every operand line is an L2 hit.  The
// results are wrong; the launch time shows what the L2 misses of the real access pattern cost.
static int diag_same_panel() {
  static const int on = [] {
    const char *e = getenv("MI355X_DIAG_SAME_PANEL");
    return (e != nullptr && e[0] == '1') ? 1 : 0;
  }();
  return on;
}

// A second one, MI355X_DIAG_KBLOCK128=<1|2|3>: builds of the 128 x 128 K-block kernel (no weight zero point, the
// one-multiply epilogue) without the operand loads after the first two K blocks (1), without the wait and the barrier
// between K blocks (2), or without both (3).  The results are wrong; the launch times say what the main loop spends
// on the matrix cores and what on feeding them.
static int diag_kblock128() {
  static const int v = [] {
    const char *e = getenv("MI355X_DIAG_KBLOCK128");
    return (e != nullptr && e[0] >= '1' && e[0] <= '3') ? e[0] - '0' : 0;
  }();
  return v;
}

template <int TILE_N, int TILE_M, int EPI, bool HAS_ZW, bool FAST, int NST = 4, int OCC = 1>
static int launch_cfg(GemmArgs g, const RequantParams &rq, const DequantParams &dq, hipStream_t stream) {
  g.tiles_m = (g.m + TILE_M - 1) / TILE_M;
  g.tiles_n = (g.n + TILE_N - 1) / TILE_N;
  const int blocks = g.tiles_m * g.tiles_n;
  auto kern = gemm_direct_kernel<TILE_N, TILE_M, EPI, HAS_ZW, FAST, NST, OCC>;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, stream, g, rq, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int EPI, bool HAS_ZW, bool FAST>
static int launch_kblock(GemmArgs g, const RequantParams &rq, const DequantParams &dq, hipStream_t stream) {
  g.tiles_m = (g.m + 255) / 256;
  g.tiles_n = (g.n + 255) / 256;
  if ((g.m & 255) != 0 || (g.n & 255) != 0) g.diag_same_panel = 0;  // (the row clamps of ragged tiles assume the tile's own base)
  hipLaunchKernelGGL((gemm_kblock_kernel<EPI, HAS_ZW, FAST>), dim3(g.tiles_m * g.tiles_n), dim3(256), 0, stream, g, rq,
                     dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int EPI, bool HAS_ZW, bool FAST>
static int launch_kblock128(GemmArgs g, const RequantParams &rq, const DequantParams &dq, hipStream_t stream) {
  g.tiles_m = (g.m + 127) / 128;
  g.tiles_n = (g.n + 127) / 128;
  if ((g.m & 127) != 0 || (g.n & 127) != 0) g.diag_same_panel = 0;
  if constexpr (!HAS_ZW && FAST) {
    if (const int d = diag_kblock128(); d != 0) {
      auto kern = d == 1   ? gemm_kblock128_diag_kernel<EPI, 1>
                  : d == 2 ? gemm_kblock128_diag_kernel<EPI, 2>
                           : gemm_kblock128_diag_kernel<EPI, 3>;
      hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(256), 0, stream, g, rq, dq);
      MI_HIP_CHECK(hipGetLastError());
      return MI_OK;
    }
  }
  hipLaunchKernelGGL((gemm_kblock128_kernel<EPI, HAS_ZW, FAST>), dim3(g.tiles_m * g.tiles_n), dim3(256), 0, stream, g,
                     rq, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int EPI, bool HAS_ZW, bool FAST>
static int launch_pick_tile(const GemmArgs &g, const RequantParams &rq, const DequantParams &dq,
                            hipStream_t stream) {
  const int64_t tiles_l = (int64_t)((g.m + 255) / 256) * ((g.n + 255) / 256);
  const int64_t tiles_m = (int64_t)((g.m + 127) / 128) * ((g.n + 127) / 128);
  // a few activation rows against a big weight matrix: one row of 64 x 64 tiles, deep prefetch (HBM-bound)
  if (g.m <= 64 && g.k_pad >= 1024) return launch_cfg<64, 64, EPI, HAS_ZW, FAST, 16>(g, rq, dq, stream);
  if (g.m <= 128 && g.k_pad >= 1024) return launch_cfg<64, 128, EPI, HAS_ZW, FAST, 8>(g, rq, dq, stream);
  // Few tiles and a long K: every workgroup walks its whole K alone at the pace of its own loop (a 64 x 64 tile takes
  // about 0.2 us per 64 bytes of K, a 64 x 128 tile 0.3, a 128 x 128 tile 0.6 per 128 bytes, whatever the number of
  // workgroups up to one per CU), so the smallest tile that still fits the device in one round wins, on eight stages
  // (three steps in flight leave a lone workgroup waiting on memory).  Measured with the weights streamed from HBM
  // (us per launch): 256 x 4096 x 4096 23.2 -> 15.6, 256 x 4096 x 11008 55.0 -> 35.7, 384 x 4096 x 4096 42.8 -> 19.5,
  // 512 x 4096 x 4096 22.2 -> 19.3, 512 x 3072 x 4096 41.2 -> 19.1, 2048 x 768 x 3072 31.8 -> 14.0,
  // 256 x 8192 x 2048 13.6 -> 12.5; with the weights in the L2s 300 x 4096 x 2048 16.4 -> 11.0,
  // 640 x 2048 x 1024 8.5 -> 6.9, and 5 % slower where fewer than a hundred tiles find them there
  // (512 x 768 x 3072: 8.5 -> 9.0).  Sixteen stages are no better than eight.
  if (g.k_pad >= 1024) {
    const int64_t cols64 = (g.n + 63) / 64;
    if ((int64_t)((g.m + 63) / 64) * cols64 <= 256) return launch_cfg<64, 64, EPI, HAS_ZW, FAST, 8, 2>(g, rq, dq, stream);
    // (against the 128 x 128 K-block tiles at K = 1024 the 64 x 128 tile is 15 % ahead on streamed weights and 4-9 %
    //  behind on cache-resident ones -- 512 x 4096 x 1024: 7.1 -> 7.7 us -- so it starts at K = 2048, where it is
    //  10-13 % ahead on those too: 512 x 4096 x 4096 20.4 -> 17.8 us, 2048 x 768 x 3072 13.9 -> 12.3 us)
    if (g.k_pad >= 2048 && (int64_t)((g.m + 127) / 128) * cols64 <= 256)
      return launch_cfg<64, 128, EPI, HAS_ZW, FAST, 8>(g, rq, dq, stream);
  }
  // The 256 x 256 tile does a unit of work in little more than half the time the 128 x 128 tiles need, so with int8
  // output it is taken as soon as the 128 x 128 tiles would no longer fit the device in one go (more than 512 of
  // them, i.e. more than 128 large tiles): 2304 x 4096 x 4096 51.6 -> 41.2 us, 2816 x 4096 x 1024 20.4 -> 17.8 us;
  // at exactly 128 large tiles the 512 small ones win (2048 x 4096 x 4096: 35.5 against 39.8 us).
  // The fp32 epilogue writes four times the bytes: below one 256 x 256 tile per CU it is worth more to overlap it
  // with another workgroup's main loop than to save operand traffic.
  // (the loader addresses activation rows with 32-bit offsets from the tile's first row)
  if (tiles_l >= (EPI == EPI_DEQUANT ? 256 : 129) && g.lda < (1 << 23))
    return launch_kblock<EPI, HAS_ZW, FAST>(g, rq, dq, stream);
  // From one 128 x 128 tile per two CUs on: the K-block loop on 128 x 128 tiles, two workgroups per CU.  Whole
  // cache lines per load and one barrier per 128 bytes of K make its main loop about a third shorter than the
  // 64-byte-step loop below; two workgroups per CU instead of three make a round of tiles more expensive.  Measured on
  // 21 int8-output shapes from 768 x 3072 x 768 to 1536 x 1536 x 6144: 0-25 % faster (2048^3 15.3 -> 13.8 us,
  // 512 x 8192 x 1024 13.8 -> 10.5 us), 2 % slower only at K = 32.  With fp32 output the epilogue weighs more: it wins
  // where the loop dominates (K >= 2048: 4096 x 768 x 3072 21.0 -> 19.0 us) and where the three-per-CU form below
  // has all its tiles store in the same moment (>= 768 tiles: 4096 x 3072 x 768 25.9 -> 24.4 us), and with at most
  // one tile per CU (4096 x 768 x 768: 8.6 -> 8.3 us); it loses on 576 tiles at K = 768 (18.4 against 22.2 us).
  if (tiles_m >= 128 && g.k >= 128 && g.lda < (1 << 23) &&
      (EPI == EPI_REQUANT || g.k >= 2048 || tiles_m >= 768 || tiles_m <= 256))
    return launch_kblock128<EPI, HAS_ZW, FAST>(g, rq, dq, stream);
  // a few hundred activation rows against many channels: 256-channel x 128-row tiles keep the weight re-reads of
  // the square 128 tile away while still giving every CU a tile
  if (g.m <= 512 && (int64_t)((g.m + 127) / 128) * ((g.n + 255) / 256) >= 128)
    return launch_cfg<256, 128, EPI, HAS_ZW, FAST>(g, rq, dq, stream);
  // the 128 x 128 tile needs a quarter of the registers and 64 KiB of LDS: two workgroups share a CU, so one tile's
  // prologue and epilogue overlap the other's main loop (what short-K shapes are made of)
  // short K and more tiles than two per CU: three stages (48 KiB) let a third workgroup in, which saves a round of
  // tiles; the shallower prefetch only costs when K is long
  if (tiles_m > 512 && g.k <= 1024) return launch_cfg<128, 128, EPI, HAS_ZW, FAST, 3, 3>(g, rq, dq, stream);
  // short K, fp32 out and fewer 128 x 128 tiles than CUs: half-width tiles, three per CU, fill the device
  if (EPI == EPI_DEQUANT && tiles_m >= 128 && tiles_m < 256 && g.k <= 1024)
    return launch_cfg<64, 128, EPI, HAS_ZW, FAST, 4, 3>(g, rq, dq, stream);
  if (tiles_m >= 128) return launch_cfg<128, 128, EPI, HAS_ZW, FAST, 4, 2>(g, rq, dq, stream);
  // (what is left has few tiles of any size; with a long K the 64 x 64 tiles take eight stages as above)
  if (g.k_pad >= 1024) return launch_cfg<64, 64, EPI, HAS_ZW, FAST, 8, 2>(g, rq, dq, stream);
  return launch_cfg<64, 64, EPI, HAS_ZW, FAST>(g, rq, dq, stream);
}

// Large fp32 outputs are written with non-temporal stores: they are not re-read out of L2 by whatever runs next, and
// they do not queue behind dirty lines.  Measured over twelve shapes with 12-75 MB of output: 3-13 % faster (BERT QKV
// 22.0 -> 19.5 us) except where every tile of the grid finishes in the same moment (exactly three tiles per CU: 2-6 %
// slower).  A compile-time choice: the two kinds of store under a run-time condition are merged into plain stores.
static bool stream_out_hint(int64_t out_bytes) { return out_bytes >= ((int64_t)8 << 20); }

static int check_args(const int8_t *a, int64_t lda, int m, int k, const WeightView &wv, int n, const void *c,
                      int64_t ldc, int c_align) {
  const int8_t *w = wv.w;
  const int k_pad = wv.k_pad;
  if (a == nullptr || w == nullptr || c == nullptr) {
    set_error("gemm: null pointer");
    return MI_NULL_PTR;
  }
  if (m <= 0 || n <= 0 || k <= 0 || (k & 15) != 0 || (lda & 15) != 0 || lda < k || k_pad % kKPad != 0 || k_pad < k ||
      wv.ldw < k_pad || (wv.ldw & 15) != 0 || (reinterpret_cast<uintptr_t>(a) & 15) != 0 || (n & 3) != 0 || (ldc & 3) != 0 || ldc < n ||
      (reinterpret_cast<uintptr_t>(c) & (c_align - 1)) != 0) {
    set_error("gemm: unsupported operand geometry m=%d n=%d k=%d lda=%lld k_pad=%d ldc=%lld", m, n, k, (long long)lda,
              k_pad, (long long)ldc);
    return MI_PARAM_INVALID;
  }
  return MI_OK;
}

int launch_gemm_requant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream) {
  int rc = check_args(a, lda, m, k, w, n, c, ldc, 4);
  if (rc != MI_OK) return rc;
  GemmArgs g{a, lda, m, k, w.w, w.ldw, w.k_pad, n, 0, 0, c, ldc, diag_same_panel()};
  DequantParams dq{};
  if (rq.has_zw) {
    return rq.fast2 ? launch_pick_tile<EPI_REQUANT, true, true>(g, rq, dq, stream)
                    : launch_pick_tile<EPI_REQUANT, true, false>(g, rq, dq, stream);
  }
  return rq.fast2 ? launch_pick_tile<EPI_REQUANT, false, true>(g, rq, dq, stream)
                  : launch_pick_tile<EPI_REQUANT, false, false>(g, rq, dq, stream);
}

template <int TILE_N, int TILE_M, bool HAS_ZW, bool FAST, int NST, int OCC>
static int launch_conv_cfg(GemmArgs g, const ConvGather &cv, const RequantParams &rq, hipStream_t stream) {
  g.tiles_m = (g.m + TILE_M - 1) / TILE_M;
  g.tiles_n = (g.n + TILE_N - 1) / TILE_N;
  auto kern = gemm_conv_kernel<TILE_N, TILE_M, HAS_ZW, FAST, NST, OCC>;
  hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(256), 0, stream, g, cv, rq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <bool HAS_ZW, bool FAST>
static int launch_conv_pick_tile(const GemmArgs &g, const ConvGather &cv, const RequantParams &rq,
                                 hipStream_t stream) {
  const int64_t tiles_m = (int64_t)((g.m + 127) / 128) * ((g.n + 127) / 128);
  // up to 64 output channels: half-width tiles (three workgroups per CU) instead of half-empty square ones
  // (more such tiles than three per CU: a fourth workgroup per CU on three stages saves the second round)
  if (g.n <= 64 && (g.m + 127) / 128 > 768) return launch_conv_cfg<64, 128, HAS_ZW, FAST, 3, 4>(g, cv, rq, stream);
  if (g.n <= 64 && g.m >= 128 * 128) return launch_conv_cfg<64, 128, HAS_ZW, FAST, 4, 3>(g, cv, rq, stream);
  if (tiles_m >= 128) return launch_conv_cfg<128, 128, HAS_ZW, FAST, 4, 2>(g, cv, rq, stream);
  return launch_conv_cfg<64, 64, HAS_ZW, FAST, 4, 1>(g, cv, rq, stream);
}

bool gemm_conv_supported(const ConvGeom &cg, const void *in, const void *out) {
  const int64_t k = (int64_t)cg.kernel_h * cg.kernel_w * cg.in_c;
  return (cg.in_c & 15) == 0 && k <= 65536 - 128 && (int64_t)cg.in_h * cg.in_w * cg.in_c < ((int64_t)1 << 31) &&
         (int64_t)cg.batch * cg.out_h * cg.out_w < ((int64_t)1 << 31) && (cg.out_c & 3) == 0 &&
         (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 3) == 0;
}

int launch_gemm_conv_requant(const int8_t *in, const ConvGeom &cg, const int8_t *fill16, const WeightView &w,
                             const RequantParams &rq, int8_t *out, hipStream_t stream) {
  const int64_t k64 = (int64_t)cg.kernel_h * cg.kernel_w * cg.in_c;
  const int64_t m64 = (int64_t)cg.batch * cg.out_h * cg.out_w;
  if (in == nullptr || fill16 == nullptr || w.w == nullptr || out == nullptr) {
    set_error("gemm_conv: null pointer");
    return MI_NULL_PTR;
  }
  if (!gemm_conv_supported(cg, in, out) || m64 <= 0 || cg.out_c <= 0 || w.k_pad % kKPad != 0 || w.k_pad < k64 ||
      w.ldw < w.k_pad || (w.ldw & 15) != 0) {
    set_error("gemm_conv: unsupported geometry ic=%d k=%lld pixels=%lld oc=%d", cg.in_c, (long long)k64,
              (long long)m64, cg.out_c);
    return MI_PARAM_INVALID;
  }
  const auto magic = [](int d) { return d <= 1 ? 0u : (uint32_t)((((uint64_t)1 << 32) + d - 1) / (uint64_t)d); };
  ConvGather cv{cg.in_h,     cg.in_w,       cg.in_c,       cg.out_w,  cg.out_h * cg.out_w, cg.kernel_w, cg.stride_h,
                cg.stride_w, cg.dilation_h, cg.dilation_w, cg.pad_u,  cg.pad_l,            magic(cg.in_c),
                magic(cg.kernel_w), fill16};
  GemmArgs g{in, 0, (int)m64, (int)k64, w.w, w.ldw, w.k_pad, cg.out_c, 0, 0, out, cg.out_c, 0};
  if (rq.has_zw) {
    return rq.fast2 ? launch_conv_pick_tile<true, true>(g, cv, rq, stream)
                    : launch_conv_pick_tile<true, false>(g, cv, rq, stream);
  }
  return rq.fast2 ? launch_conv_pick_tile<false, true>(g, cv, rq, stream)
                  : launch_conv_pick_tile<false, false>(g, cv, rq, stream);
}

int launch_gemm_dequant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const DequantParams &dq, float *c, int64_t ldc, hipStream_t stream) {
  int rc = check_args(a, lda, m, k, w, n, c, ldc, 16);
  if (rc != MI_OK) return rc;
  GemmArgs g{a, lda, m, k, w.w, w.ldw, w.k_pad, n, 0, 0, c, ldc, diag_same_panel()};
  RequantParams rq{};
  // the third parameter (the fast-rounding switch of the int8 epilogue) selects non-temporal stores here
  const bool nt = stream_out_hint((int64_t)m * n * 4);
  if (dq.zw0 != 0) {
    return nt ? launch_pick_tile<EPI_DEQUANT, true, true>(g, rq, dq, stream)
              : launch_pick_tile<EPI_DEQUANT, true, false>(g, rq, dq, stream);
  }
  return nt ? launch_pick_tile<EPI_DEQUANT, false, true>(g, rq, dq, stream)
            : launch_pick_tile<EPI_DEQUANT, false, false>(g, rq, dq, stream);
}

}  // namespace mi
