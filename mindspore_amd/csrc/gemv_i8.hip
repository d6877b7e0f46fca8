// Skinny-M (decode) int8 GEMV with the requantising epilogue of the full-quant MatMul: M <= 64 activation rows
// against the packed int8 weight matrix (n_pad rows of k_pad bytes, row stride ldw): a v_dot4 kernel for one row (and
// for two on a handle without the blocked weight copy), matrix-core kernels on the blocked copy for 2 <= M <= 64.
// The kernels are HBM-bound on the weight stream, so the design goal is "every weight byte crosses HBM once, in 1 KiB
// coalesced wave loads, with enough loads in flight":
//   - v_dot4 kernel: a wave owns R consecutive output channels and walks K in 1 KiB segments (64 lanes x 16 bytes),
//     with its whole share in flight where that fits (D 16-byte loads per lane); the K reduction across lanes happens
//     once at the end;
//   - matrix-core kernels: a workgroup of eight waves owns RG x 16 channels, the waves split K, the weights are the
//     16-row operand of v_mfma_i32_16x16x64_i8 and are read from 1 KiB blocks laid out in lane order; the activation
//     rows go through LDS.
// Arithmetic reference: MatmulInt8Opt, mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/matmul_int8.c:296-331.
#include "common.h"
#include "quant_math.h"

#include <algorithm>
#include <cstdlib>
#include <type_traits>


namespace mi {

typedef int v4i __attribute__((ext_vector_type(4)));

// Sum over the 64 lanes of a wave, returned as a wave-uniform value: DPP adds inside each row of 16 lanes
// (quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_ror:4, row_ror:8), then one lane per row is read back.
__device__ __forceinline__ int wave_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x124, 0xF, 0xF, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, false);
  return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
         __builtin_amdgcn_readlane(v, 48);
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
  int ldw;    // weight row stride in bytes
  int k_pad;  // contraction extent of a (zero padded) weight row
  int n;
  int8_t *c;
  int64_t ldc;
};

// One wave owns R consecutive output channels and walks its R x K weight bytes as a stream of 1 KiB chunks
// (chunk c = K segment c / R of row c % R, so one activation fragment serves R consecutive chunks).  D chunks are
// in flight: a register slot is refilled with the chunk D positions ahead as soon as it has been consumed.  When
// R * ceil(K / 1 KiB) <= D the whole share of the wave is requested up front and nothing loops.
// No weight load is predicated (a predicated load makes the compiler wait for earlier loads before issuing later
// ones): lanes past the end of a row re-read its last 16 bytes and chunks past the end of the stream re-read the
// last chunk; both meet a zero activation fragment or are not accumulated.
// KS = 2: two neighbouring waves share their R rows, each walks one half of K (long rows: twice the waves, each with
// half the registers, so that more of them are resident), and the even wave adds the odd wave's sums through LDS.
// DEQ: the fp32 epilogue of the dynamic-quant MatMul (see gemv_mfma_lds_body) instead of the requantising one.
template <int M, int R, int D, bool DIRECT, int KS, bool DEQ = false>
__device__ __forceinline__ void gemv_i8_body(const GemvArgs &g, const RequantParams &rq, const DequantParams &dq,
                                             int block) {
  const bool has_zw = DEQ ? dq.zw0 != 0 : rq.has_zw != 0;
  static_assert(D % R == 0, "the slot -> row mapping must be static");
  static_assert(KS == 1 || KS == 2, "one or two waves per row group");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  v4i *sa = reinterpret_cast<v4i *>(smem);  // [M][nseg_all * 64], zero past K
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_base = (block * (4 / KS) + wave / KS) * R;
  const int nseg_all = (g.kchunks + 63) >> 6;
  const int kc_pad = nseg_all * 64;
  const int seg_per = (nseg_all + KS - 1) / KS;
  const int seg0 = (wave % KS) * seg_per;                                   // this wave's K segments: seg0 ..
  const int nseg = seg0 < nseg_all ? (seg_per < nseg_all - seg0 ? seg_per : nseg_all - seg0) : 0;  // .. seg0 + nseg
  const int total = nseg * R;
  const int last_off = (g.kchunks - 1) * 16;
  const int8_t *wrow = g.w + (int64_t)n_base * g.ldw;

  // (a slot past the end of the stream -- only the looping form has such -- asks for the first 16 bytes of the
  //  activation row, which are in the nearest cache, instead of pulling weight bytes through the memory system again)
  auto load_chunk = [&](int c) -> v4i {
    const bool live = c < total;
    c = live ? c : 0;
    const int seg = seg0 + c / R, rr = c % R;
    int off = seg * 1024 + lane * 16;
    off = off < last_off ? off : last_off;
    const int8_t *p = live ? wrow + (int64_t)rr * g.ldw + off : g.a;
    return __builtin_nontemporal_load(reinterpret_cast<const v4i *>(p));
  };
  v4i buf[D];
#pragma unroll
  for (int i = 0; i < D; ++i) buf[i] = load_chunk(i);
  // lane rr*M + m finishes output (m, n_base + rr): fetch its channel's parameters now, so their latency hides
  // behind the weight stream (the parameter arrays are padded to a multiple of 256 channels)
  const int my_rr = lane / M, my_m = lane - my_rr * M;
  const int my_n = n_base + (lane < R * M ? my_rr : 0);
  int32_t p_mult = 0, p_e = 0, p_ls = 0, p_bias2 = 0, p_zw = 0, d_wsum = 0, d_zx = 0;
  float d_ws = 0.0f, d_bias = 0.0f, d_sx = 0.0f;
  if (DEQ) {
    d_ws = dq.wscale[my_n];
    d_wsum = dq.wsum[my_n];
    // The optional operands are fetched unconditionally, from an address that is valid either way, and selected
    // afterwards: a conditional fetch is a branch, and behind those branches the compiler waited for every outstanding
    // load after each of the activation fetches below (six round trips in a row: 4096 x 11008 at one row 10.9 us
    // against 9.0 for the requantising form of the same kernel).
    const bool on_dev = dq.qp_dev != nullptr;
    const float *bias_or_any = dq.bias != nullptr ? dq.bias : dq.wscale;
    const mi_dq_params *qp_or_any = on_dev ? dq.qp_dev : reinterpret_cast<const mi_dq_params *>(dq.wscale);
    d_bias = bias_or_any[my_n];
    const float sx_dev = qp_or_any[on_dev && dq.per_row && lane < R * M ? my_m : 0].scale_f;
    const int32_t zx_dev = qp_or_any->zero_point;
    d_sx = on_dev ? sx_dev : dq.sx;
    d_zx = on_dev ? zx_dev : dq.zx;
  } else {
    p_mult = rq.mult[my_n];
    p_e = rq.rshift[my_n];
    p_ls = rq.lshift[my_n];
    p_bias2 = rq.bias2[my_n];
    p_zw = rq.zw[my_n];
  }

  // DIRECT (the whole share of the wave is in flight, total <= D): every wave fetches its own activation fragments
  // straight into registers -- no LDS, no workgroup barrier.  Otherwise the workgroup stages the activations in LDS
  // once (the weight loads above are already in flight either way).
  // The fp32 form fetches them through a buffer descriptor (a fetch whose lane offset is out of range returns zeros
  // without touching memory, so chunks past K and segments past the wave's share need no substitute address and no
  // mask on the data): with masks on the data the compiler had, in that form, waited for each fetch before issuing the
  // next -- six round trips in a row, 4096 x 11008 at one row 10.9 us against 9.0 for the requantising form, whose
  // fetches it issues together.  That form keeps the masks: with the descriptor it measured 2 % slower over a decoder
  // layer (5.36 against 5.46 TB/s).
  v4i apre[DIRECT ? D / R : 1][M];
  if (DIRECT) {
    constexpr int kOutOfRange = (int)0x80000000u;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(g.a), (short)0, (int)((M - 1) * g.lda) + g.kchunks * 16, 0x00020000);
#pragma unroll
    for (int sgi = 0; sgi < D / R; ++sgi)
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const int chunk = (seg0 + sgi) * 64 + lane;
        const bool live = chunk < g.kchunks && sgi < nseg;
        if constexpr (DEQ) {
          apre[sgi][m] = __builtin_bit_cast(
              v4i, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, live ? m * (int)g.lda + chunk * 16 : kOutOfRange, 0, 0));
        } else {
          const int cc = chunk < g.kchunks ? chunk : g.kchunks - 1;
          const v4i v = reinterpret_cast<const v4i *>(g.a + (int64_t)m * g.lda)[cc];
          apre[sgi][m].x = live ? v.x : 0;
          apre[sgi][m].y = live ? v.y : 0;
          apre[sgi][m].z = live ? v.z : 0;
          apre[sgi][m].w = live ? v.w : 0;
        }
      }
  } else {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const v4i *arow = reinterpret_cast<const v4i *>(g.a + (int64_t)m * g.lda);
      for (int ch = tid; ch < kc_pad; ch += 256) {
        v4i z = {0, 0, 0, 0};
        sa[m * kc_pad + ch] = ch < g.kchunks ? arow[ch] : z;
      }
    }
    __syncthreads();
  }

  int acc[R][M];
  int asum[M];
#pragma unroll
  for (int rr = 0; rr < R; ++rr)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[rr][m] = 0;
#pragma unroll
  for (int m = 0; m < M; ++m) asum[m] = 0;

  v4i af[M];
  auto pass = [&](int base, auto refill) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      const int c = base + i;
      const v4i w = buf[i];
      if (decltype(refill)::value) buf[i] = load_chunk(c + D);
      if (i % R == 0) {  // first row of a K segment: fetch the activation fragments for it (zero past the stream)
        if (M > 2) __builtin_amdgcn_sched_barrier(0);  // keeps the fragments of later segments out of registers
        const int seg = c / R;
#pragma unroll
        for (int m = 0; m < M; ++m) {
          v4i z = {0, 0, 0, 0};
          if (DIRECT) {
            af[m] = apre[i / R][m];
          } else {
            af[m] = seg < nseg ? sa[m * kc_pad + (seg0 + seg) * 64 + lane] : z;
          }
          if (has_zw) {
            v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
            asum[m] = dot16(af[m], ones, asum[m]);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < M; ++m) acc[i % R][m] = dot16(w, af[m], acc[i % R][m]);
    }
  };
  int base = 0;
  for (; base + D < total; base += D) pass(base, std::true_type());
  pass(base, std::false_type());

  // reduce over lanes (wave-uniform totals); lane rr*M + m keeps the one it finishes
  int mine = 0, my_asum = 0;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    int s = 0;
    if (has_zw) s = wave_sum(asum[m]);
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
      const int t = wave_sum(acc[rr][m]);
      if (lane == rr * M + m) {
        mine = t;
        my_asum = s;
      }
    }
  }
  if (KS == 2) {
    __shared__ int halves[2][2][64];  // [row group of the workgroup][sum, activation sum][lane]
    if (wave & 1) {
      halves[wave >> 1][0][lane] = mine;
      halves[wave >> 1][1][lane] = my_asum;
    }
    __syncthreads();
    if (wave & 1) return;
    mine += halves[wave >> 1][0][lane];
    my_asum += halves[wave >> 1][1][lane];
  }
  if (lane < R * M) {
    const int m = my_m, n = my_n;
    if (n < g.n && DEQ) {
      uint32_t v = (uint32_t)mine;
      v += (uint32_t)dq.deep * (uint32_t)d_zx * (uint32_t)dq.zw0 - (uint32_t)d_zx * (uint32_t)d_wsum;
      if (has_zw) v -= (uint32_t)dq.zw0 * (uint32_t)my_asum;
      float d = __fmul_rn(__fmul_rn(d_sx, d_ws), (float)(int32_t)v);
      if (dq.bias != nullptr) d = __fadd_rn(d, d_bias);
      const bool with_act = dq.act == MI_ACT_RELU || dq.act == MI_ACT_RELU6;
      const float act_lo = with_act ? 0.0f : -__builtin_inff();
      const float act_hi = dq.act == MI_ACT_RELU6 ? 6.0f : __builtin_inff();
      d = (act_lo > d) ? act_lo : d;
      d = (act_hi < d) ? act_hi : d;
      reinterpret_cast<float *>(g.c)[(int64_t)m * g.ldc + n] = d;
    } else if (n < g.n) {
      uint32_t v = (uint32_t)mine;
      if (has_zw) v -= (uint32_t)my_asum * (uint32_t)p_zw;
      v += (uint32_t)p_bias2;
      const int32_t mult = p_mult, e = p_e;
      int32_t y;
      if (rq.fast) {
        y = rdiv_pot_fast(srdhm_nosat((int32_t)v, mult), e, (1 << e) >> 1);
      } else {
        y = rdiv_pot(srdhm((int32_t)(v << p_ls), mult), e);
      }
      y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
      y = y < rq.amax ? y : rq.amax;
      y = y > rq.amin ? y : rq.amin;
      g.c[(int64_t)m * g.ldc + n] = (int8_t)y;
    }
  }
}

template <int M, int R, int D, bool DIRECT, int KS>
__global__ __launch_bounds__(256) void gemv_i8_kernel(GemvArgs g, RequantParams rq) {
  gemv_i8_body<M, R, D, DIRECT, KS, false>(g, rq, DequantParams{}, (int)blockIdx.x);
}

template <int M, int R, int D, bool DIRECT, int KS>
__global__ __launch_bounds__(256) void gemv_i8_deq_kernel(GemvArgs g, DequantParams dq) {
  gemv_i8_body<M, R, D, DIRECT, KS, true>(g, RequantParams{}, dq, (int)blockIdx.x);
}

// Several weight matrices against the same activation rows in one launch (MatMuls that share their input, e.g. the
// gate and up projections of a decoder layer): the grid is the concatenation of the members' grids, and a workgroup
// first finds the member it belongs to.  Every field is picked with selects over constant indices, which keeps the
// table in scalar registers (a dynamically indexed kernel argument would be copied to scratch memory).
constexpr int kGemvGroupMax = 4;
template <typename P>  // P: the members' epilogue parameters (RequantParams or DequantParams)
struct GemvGroupT {
  int count;
  int block_end[kGemvGroupMax];  // exclusive prefix sums of the members' workgroup counts
  GemvArgs g[kGemvGroupMax];
  P rq[kGemvGroupMax];
};
typedef GemvGroupT<RequantParams> GemvGroup;
typedef GemvGroupT<DequantParams> GemvGroupDeq;

template <typename P>
__device__ __forceinline__ void pick_member(const GemvGroupT<P> &grp, int block, GemvArgs *g, P *rq,
                                            int *local_block) {
  int member = 0;
#pragma unroll
  for (int i = 1; i < kGemvGroupMax; ++i)
    if (i < grp.count && block >= grp.block_end[i - 1]) member = i;
  *g = grp.g[0];
  *rq = grp.rq[0];
  *local_block = block;
#pragma unroll
  for (int i = 1; i < kGemvGroupMax; ++i) {
    if (member == i) {
      *g = grp.g[i];
      *rq = grp.rq[i];
      *local_block = block - grp.block_end[i - 1];
    }
  }
}

template <int M, int R, int D, bool DIRECT, int KS>
__global__ __launch_bounds__(256) void gemv_i8_group_kernel(GemvGroup grp) {
  GemvArgs g;
  RequantParams rq;
  int block;
  pick_member(grp, (int)blockIdx.x, &g, &rq, &block);
  gemv_i8_body<M, R, D, DIRECT, KS, false>(g, rq, DequantParams{}, block);
}

template <int M, int R, int D, bool DIRECT, int KS>
__global__ __launch_bounds__(256) void gemv_i8_group_deq_kernel(GemvGroupDeq grp) {
  GemvArgs g;
  DequantParams dq;
  int block;
  pick_member(grp, (int)blockIdx.x, &g, &dq, &block);
  gemv_i8_body<M, R, D, DIRECT, KS, true>(g, RequantParams{}, dq, block);
}

template <int M, int R, int D, bool DIRECT, int KS>
static int launch_mrdx(const GemvArgs &g, const RequantParams &rq, hipStream_t stream) {
  auto kern = gemv_i8_kernel<M, R, D, DIRECT, KS>;
  // (more than 64 KiB of dynamic LDS needs the attribute that gemv_prepare_device set when the library was initialised)
  const int lds_bytes = DIRECT ? 0 : M * ((g.kchunks + 63) / 64) * 1024;
  const int rows_per_block = 4 / KS * R;
  const int blocks = (g.n + rows_per_block - 1) / rows_per_block;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds_bytes, stream, g, rq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int M, int R, int D, bool DIRECT, int KS>
static int launch_mrdx_deq(const GemvArgs &g, const DequantParams &dq, hipStream_t stream) {
  const int lds_bytes = DIRECT ? 0 : M * ((g.kchunks + 63) / 64) * 1024;
  const int rows_per_block = 4 / KS * R;
  const int blocks = (g.n + rows_per_block - 1) / rows_per_block;
  hipLaunchKernelGGL((gemv_i8_deq_kernel<M, R, D, DIRECT, KS>), dim3(blocks), dim3(256), lds_bytes, stream, g, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int M, int R, int D, bool DIRECT, int KS, typename P>
static int launch_group_mrdx(GemvGroupT<P> &grp, hipStream_t stream) {
  const int lds_bytes = DIRECT ? 0 : M * ((grp.g[0].kchunks + 63) / 64) * 1024;
  int blocks = 0;
  for (int i = 0; i < grp.count; ++i) {
    blocks += (grp.g[i].n + 4 / KS * R - 1) / (4 / KS * R);
    grp.block_end[i] = blocks;
  }
  if constexpr (std::is_same<P, DequantParams>::value) {
    hipLaunchKernelGGL((gemv_i8_group_deq_kernel<M, R, D, DIRECT, KS>), dim3(blocks), dim3(256), lds_bytes, stream, grp);
  } else {
    hipLaunchKernelGGL((gemv_i8_group_kernel<M, R, D, DIRECT, KS>), dim3(blocks), dim3(256), lds_bytes, stream, grp);
  }
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int M>
static int allow_big_lds() {
  // the looping form stages the activation rows in dynamic LDS: up to 160 KiB
  MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_i8_kernel<M, 1, 12, false, 1>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_i8_group_kernel<M, 1, 12, false, 1>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  if (M == 1) {
    MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_i8_deq_kernel<1, 1, 12, false, 1>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gemv_i8_group_deq_kernel<1, 1, 12, false, 1>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  }
  return MI_OK;
}

// Once per device, from mi_init.
int gemv_prepare_device() {
  int rc;
  if ((rc = allow_big_lds<1>()) != MI_OK || (rc = allow_big_lds<2>()) != MI_OK) return rc;
  return MI_OK;
}

// Measured on MI355X: HBM streams fastest with many light waves that each have their whole share in flight at once
// (a wave that loops needs >= 8-16 resident waves per CU to keep up), and a load slot that has no chunk of its own
// still costs a request.  So rows per wave R and slots D are picked so that R x ceil(K / 1 KiB) == D exactly for
// every K up to 12 KiB; longer rows loop over 12 slots with the activation rows staged in LDS.
template <int M, typename F>
static int with_config(int nseg, F &&f) {
  using std::integral_constant;
  typedef integral_constant<int, 1> one;
  typedef integral_constant<int, 2> two;
  switch (nseg) {  // f(R, D, DIRECT, KS)
    case 1: return f(integral_constant<int, 4>(), integral_constant<int, 4>(), std::true_type(), one());
    case 2: return f(integral_constant<int, 4>(), integral_constant<int, 8>(), std::true_type(), one());
    case 3: return f(two(), integral_constant<int, 6>(), std::true_type(), one());
    case 4: return f(two(), integral_constant<int, 8>(), std::true_type(), one());
    case 5: return f(two(), integral_constant<int, 10>(), std::true_type(), one());
    case 6: return f(two(), integral_constant<int, 12>(), std::true_type(), one());
    // from here on the rows are long enough that one per wave would need 7+ KiB of slots plus as many activation
    // registers: two waves per row, each with half of K
    case 7:
    case 8: return f(one(), integral_constant<int, 4>(), std::true_type(), two());
    case 9:
    case 10: return f(one(), integral_constant<int, 5>(), std::true_type(), two());
    case 11:
    case 12: return f(one(), integral_constant<int, 6>(), std::true_type(), two());
    default: return f(one(), integral_constant<int, 12>(), std::false_type(), one());
  }
}

template <int M, typename P>
static int launch_group_m(GemvGroupT<P> &grp, hipStream_t stream) {  // the choice depends on K only
  return with_config<M>((grp.g[0].kchunks + 63) >> 6, [&](auto r, auto d, auto direct, auto ks) {
    return launch_group_mrdx<M, decltype(r)::value, decltype(d)::value, decltype(direct)::value, decltype(ks)::value>(
        grp, stream);
  });
}

template <int M>
static int launch_m(const GemvArgs &g, const RequantParams &rq, hipStream_t stream) {
  return with_config<M>((g.kchunks + 63) >> 6, [&](auto r, auto d, auto direct, auto ks) {
    return launch_mrdx<M, decltype(r)::value, decltype(d)::value, decltype(direct)::value, decltype(ks)::value>(
        g, rq, stream);
  });
}

// =====================================================================================================================
// 2 <= M <= 64 activation rows: the matrix cores do the products, so the arithmetic cost does not grow with M.
// v_mfma_i32_16x16x64_i8 with the WEIGHTS as the 16-row operand: lane (g = lane / 16, i = lane % 16) supplies 16
// contiguous K bytes of weight row i (K offset 16 g inside the 64-byte step) and the same 16 K bytes of activation row
// i (zero for i >= M; rows 16..31, 32..47 and 48..63 are further fragments against the same weight fragment); the result register r of
// that lane is output (channel 4 g + r, activation row i).
// The weights come from the blocked copy: 1 KiB blocks [row / 16][k / 64], inside a block the 16-byte chunks in lane
// order ([(k % 64) / 16][row % 16]), so a wave instruction fetches 64 consecutive chunks -- eight whole cache lines --
// and a wave's consecutive steps walk consecutive KiB.  (With the chunks in row order the same KiB cost four times
// the cache-line lookups, and the decode matrices ran 10-20 % slower.)
// A workgroup of 8 waves owns RG x 16 channels; the waves split K into contiguous slices, each wave keeps D steps
// (D x RG KiB of weights) in flight.
//
// The activation rows go through LDS.  Fetched straight into fragments, an instruction asks for 64 bytes of each of
// up to 16 rows: four lanes per row, so every group of four neighbouring lanes touches four different cache lines, and
// the address unit looks a line up per lane group rather than per instruction.  Instead a wave fetches its K slice of
// the rows with lanes along K (the MR x D x 64 bytes of a pass as MR runs of whole cache lines), writes them to a
// private LDS area one row after the other (row stride D x 64 + 16 bytes, so that the 16 rows of a fragment read fall
// on different banks) and reads the fragments back from there.  Row MR of the area stays zero: lanes whose row does
// not exist read it.  The area is private to the wave (LDS operations of one wave execute in order), so staging needs
// no barrier.
// Both operands are fetched through buffer descriptors, so a fetch that has nothing to fetch returns zeros without a
// memory access and without a mask on the data.
// The waves' partial sums meet in LDS accumulators (atomic adds), and after one barrier every wave finishes one
// (activation row group, channel group, result register) triple, one output per lane: the barrier and what follows it
// is what a launch with one workgroup per CU cannot overlap with anything, so it is kept short (measured on the decode
// matrices at 8 rows: 0.1-0.3 us per launch against eight partial reads per output by the first waves only).
// RG channel groups per workgroup: activation bytes per weight byte are M / (16 RG); three where there are channels
// enough (a 12288 x 4096 matrix is then 256 workgroups, one per CU, all resident at once).  MR = the number of rows
// rounded up to 2, 4, 8, 16, 32 or 64 (the number of fetch instructions is a compile-time constant).
// Measured over a decoder layer against fragments fetched from global memory, eight partial reads per output and two
// channel groups: 8 rows 4.57 -> 4.95 TB/s, 16 rows 3.95 -> 4.58, 32 rows 2.67 -> 3.66.
// =====================================================================================================================
// DIAG: timing what-ifs (wrong results, see gemv_diag()): bit 0 = no activation fetches, bit 1 = no barrier before the
// final sum.
// DEQ: the fp32 epilogue of the dynamic-quant MatMul (DynamicMatmul4x16x4AIWI,
// mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/dynamic_matmul_int8.c:99-143) instead of the requantising one:
// value = sum - zx * sum_k w - zw * sum_k a + K * zx * zw, out = (sx[row] * sw[c]) * (float)value (+ bias) (activation);
// g.c then points at floats.
template <int WAVES, int RG, int D, int MR, int DIAG = 0, bool DEQ = false>
__device__ __forceinline__ void gemv_mfma_lds_body(const GemvArgs &g, int m_rows, const RequantParams &rq,
                                                   const DequantParams &dq, int block) {
  const bool has_zw = DEQ ? dq.zw0 != 0 : rq.has_zw != 0;
  constexpr int ROWB = D * 64;                       // activation bytes per row and pass
  constexpr int STRIDE = ROWB + 16;                  // LDS row stride
  constexpr int LPR = ROWB / 16;                     // 16-byte chunks of one row in a pass
  constexpr int NLD = (MR * LPR + 63) / 64;          // fetch instructions per pass
  constexpr int AREA = (MR + 1) * STRIDE;            // per wave
  constexpr int MG = MR > 16 ? MR / 16 : 1;          // groups of 16 activation rows
  constexpr int NSUM = (4 * RG + 1) * MG;            // accumulators per lane: 4 RG results + the row sum, per row group
  __shared__ int sums[NSUM * 64];
  __shared__ __attribute__((aligned(16))) char lds[WAVES * AREA];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = lane >> 4, idx = lane & 15;
  const int n0 = block * (RG * 16);
  const int k_bytes = g.kchunks * 16;
  const int total = g.k_pad >> 6;  // 64-byte steps in a (zero padded) weight row
  const int spw = (total + WAVES - 1) / WAVES;
  const int s0 = wave * spw;
  char *area = lds + wave * AREA;
  const int n_pad = (g.n + 255) & ~255;            // rows of the packed weights and of the parameter arrays
  const int rg_live = (n_pad - n0) >> 4;           // row groups of this workgroup that exist (RG need not divide 16)

  // Both operands come through buffer descriptors: a load whose lane offset is kOutOfRange returns zero without touching
  // memory, so loads that have nothing to fetch (a step past the wave's slice or past the row, a row group or an
  // activation row that does not exist, bytes past K) need neither a substitute address nor a mask on the data, and a
  // load's address is one lane offset plus a scalar.
  constexpr int kOutOfRange = (int)0x80000000u;
  const int sw0 = __builtin_amdgcn_readfirstlane(s0);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<int8_t *>(g.w) + (int64_t)(n0 >> 4) * total * 1024, (short)0,
      (rg_live < RG ? rg_live : RG) * total * 1024, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<int8_t *>(g.a), (short)0, (int)((m_rows - 1) * g.lda) + k_bytes, 0x00020000);
  // fetch geometry: the MR x LPR chunks of a pass in row-major order, 64 per instruction
  int a_off[NLD], a_chunk[NLD], a_dst[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int c = i * 64 + lane, row = c / LPR, chunk = c % LPR;
    a_chunk[i] = chunk;
    a_off[i] = row < m_rows ? row * (int)g.lda + chunk * 16 : kOutOfRange;
    a_dst[i] = row < MR ? row * STRIDE + chunk * 16 : -1;
  }
  auto load_a = [&](int base, int i) -> v4i {
    const int step = base + (a_chunk[i] >> 2);
    const int kb = (sw0 + base) * 64;
    const bool any = base < spw && sw0 + base < total && kb < k_bytes;  // (wave-uniform)
    const bool live = step < spw && sw0 + step < total && kb + a_chunk[i] * 16 < k_bytes;
    return __builtin_bit_cast(
        v4i, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, live ? a_off[i] : kOutOfRange, any ? kb : 0, 0));
  };
  auto store_a = [&](int base, int i, v4i v) {
    if (a_dst[i] >= 0) *reinterpret_cast<v4i *>(area + a_dst[i]) = v;
  };
  auto load_w = [&](int j, int rg) -> v4i {
    const int s = sw0 + j;
    const bool live = j < spw && s < total && rg < rg_live;  // (wave-uniform)
    return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, live ? lane * 16 : kOutOfRange,
                                                                         live ? (rg * total + s) * 1024 : 0, 2));
  };

  // activations first: they return first, and the rows can be in LDS while the weights are still on their way
  constexpr bool kFetchA = (DIAG & 1) == 0, kMeet = (DIAG & 2) == 0;
  v4i abuf[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) abuf[i] = kFetchA ? load_a(0, i) : v4i{lane, 1, 2, 3};
  v4i wbuf[D][RG];
#pragma unroll
  for (int j = 0; j < D; ++j)
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) wbuf[j][rg] = load_w(j, rg);
  for (int c = lane; c < STRIDE / 16; c += 64) *reinterpret_cast<v4i *>(area + MR * STRIDE + c * 16) = v4i{0, 0, 0, 0};
  for (int c = tid; c < NSUM * 64; c += WAVES * 64) sums[c] = 0;
  __syncthreads();  // (every wave gets here right after it has issued its loads)

  // after the reduction, (activation row group, channel group, result register) triple q = wave + 8 t is finished by
  // this wave: one output per lane and triple
  constexpr int NQ = (4 * RG * MG + WAVES - 1) / WAVES;
  int32_t p_mult[NQ], p_e[NQ], p_ls[NQ], p_bias2[NQ], p_zw[NQ];
  float d_ws[NQ], d_bias[NQ], d_sx[NQ];  // DEQ: weight scale, fp32 bias, input scale of the lane's row
  int32_t d_wsum[NQ], d_zx = 0;
#pragma unroll
  for (int t = 0; t < NQ; ++t) {
    const int qq = wave + WAVES * t;
    const int q = qq % (4 * RG);  // (the channel does not depend on the activation row group)
    const int n = (q >> 2) < rg_live ? n0 + (q >> 2) * 16 + 4 * grp + (q & 3) : n0;
    if (DEQ) {
      d_ws[t] = dq.wscale[n];
      d_wsum[t] = dq.wsum[n];
      d_bias[t] = dq.bias != nullptr ? dq.bias[n] : 0.0f;
      int row = idx + 16 * (qq / (4 * RG));
      row = row < m_rows ? row : m_rows - 1;
      d_sx[t] = dq.qp_dev != nullptr ? dq.qp_dev[dq.per_row ? row : 0].scale_f : dq.sx;
    } else {
      p_mult[t] = rq.mult[n];
      p_e[t] = rq.rshift[n];
      p_ls[t] = rq.lshift[n];
      p_bias2[t] = rq.bias2[n];
      p_zw[t] = rq.zw[n];
    }
  }
  if (DEQ) d_zx = dq.qp_dev != nullptr ? dq.qp_dev->zero_point : dq.zx;

  v4i acc[MG][RG], asum[MG];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) {
    asum[mg] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) acc[mg][rg] = v4i{0, 0, 0, 0};
  }
  const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
  const char *frag[MG];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) frag[mg] = area + (idx + 16 * mg < m_rows ? idx + 16 * mg : MR) * STRIDE + grp * 16;

  auto pass = [&](int base, auto refill) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) store_a(base, i, abuf[i]);
    if (decltype(refill)::value && kFetchA) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) abuf[i] = load_a(base + D, i);
    }
#pragma unroll
    for (int j = 0; j < D; ++j) {
      v4i x[MG];
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) x[mg] = *reinterpret_cast<const v4i *>(frag[mg] + j * 64);
      // (the slot is refilled before the products that read its old contents: the new fetch gets registers of its
      //  own and does not have to wait for the old data, so a wave has up to two passes in flight; refilling after
      //  the products saves a third of the registers and costs 5 % of the decode rate)
      v4i w[RG];
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) w[rg] = wbuf[j][rg];
      if (decltype(refill)::value) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg) wbuf[j][rg] = load_w(base + D + j, rg);
      }
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) {
#pragma unroll
        for (int rg = 0; rg < RG; ++rg)
          acc[mg][rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[rg], x[mg], acc[mg][rg], 0, 0, 0);
        if (has_zw) asum[mg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, x[mg], asum[mg], 0, 0, 0);
      }
    }
  };
  int base = 0;
  for (; base + D < spw; base += D) pass(base, std::true_type());
  pass(base, std::false_type());

  // the partial sums meet in LDS accumulators (LDS atomic adds without a return value; the accumulators were zeroed
  // before the first barrier): for activation row group mg, register r of channel group rg at
  // sums[((4 RG + 1) mg + 4 rg + r) * 64 + lane], the row sum behind them
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) {
    int *dst = sums + (4 * RG + 1) * mg * 64 + lane;
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        __hip_atomic_fetch_add(dst + (4 * rg + r) * 64, acc[mg][rg][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (has_zw)
      __hip_atomic_fetch_add(dst + 4 * RG * 64, asum[mg][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  if (kMeet) __syncthreads();
#pragma unroll
  for (int t = 0; t < NQ; ++t) {
    const int qq = wave + WAVES * t;
    const int mg = qq / (4 * RG), q = qq % (4 * RG);
    const int f_n = n0 + (q >> 2) * 16 + 4 * grp + (q & 3);
    const int row = idx + 16 * mg;
    if (qq < 4 * RG * MG && row < m_rows && f_n < g.n) {
      const int *src = sums + (4 * RG + 1) * mg * 64 + lane;
      uint32_t v = (uint32_t)src[q * 64];
      if (DEQ) {
        // the steps of the reference, separately rounded: int -> float, the scale product, the product, the bias
        v += (uint32_t)dq.deep * (uint32_t)d_zx * (uint32_t)dq.zw0 - (uint32_t)d_zx * (uint32_t)d_wsum[t];
        if (has_zw) v -= (uint32_t)dq.zw0 * (uint32_t)src[4 * RG * 64];
        float d = __fmul_rn(__fmul_rn(d_sx[t], d_ws[t]), (float)(int32_t)v);
        if (dq.bias != nullptr) d = __fadd_rn(d, d_bias[t]);
        // (bounds that are infinite where the reference makes no comparison: false for every d, NaN included)
        const bool with_act = dq.act == MI_ACT_RELU || dq.act == MI_ACT_RELU6;
        const float act_lo = with_act ? 0.0f : -__builtin_inff();
        const float act_hi = dq.act == MI_ACT_RELU6 ? 6.0f : __builtin_inff();
        d = (act_lo > d) ? act_lo : d;
        d = (act_hi < d) ? act_hi : d;
        reinterpret_cast<float *>(g.c)[(int64_t)row * g.ldc + f_n] = d;
      } else {
        if (has_zw) v -= (uint32_t)src[4 * RG * 64] * (uint32_t)p_zw[t];
        v += (uint32_t)p_bias2[t];
        int32_t y;
        if (rq.fast) {
          y = rdiv_pot_fast(srdhm_nosat((int32_t)v, p_mult[t]), p_e[t], (1 << p_e[t]) >> 1);
        } else {
          y = rdiv_pot(srdhm((int32_t)(v << p_ls[t]), p_mult[t]), p_e[t]);
        }
        y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
        y = y < rq.amax ? y : rq.amax;
        y = y > rq.amin ? y : rq.amin;
        g.c[(int64_t)row * g.ldc + f_n] = (int8_t)y;
      }
    }
  }
}

template <int WAVES, int RG, int D, int MR, int DIAG = 0>
__global__ __launch_bounds__(WAVES * 64) void gemv_mfma_lds_kernel(GemvArgs g, int m_rows, RequantParams rq) {
  gemv_mfma_lds_body<WAVES, RG, D, MR, DIAG, false>(g, m_rows, rq, DequantParams{}, (int)blockIdx.x);
}

template <int WAVES, int RG, int D, int MR>
__global__ __launch_bounds__(WAVES * 64) void gemv_mfma_lds_deq_kernel(GemvArgs g, int m_rows, DequantParams dq) {
  gemv_mfma_lds_body<WAVES, RG, D, MR, 0, true>(g, m_rows, RequantParams{}, dq, (int)blockIdx.x);
}

template <int WAVES, int RG, int D, int MR>
__global__ __launch_bounds__(WAVES * 64) void gemv_mfma_lds_group_kernel(GemvGroup grp, int m_rows) {
  GemvArgs g;
  RequantParams rq;
  int block;
  pick_member(grp, (int)blockIdx.x, &g, &rq, &block);
  gemv_mfma_lds_body<WAVES, RG, D, MR, 0, false>(g, m_rows, rq, DequantParams{}, block);
}

template <int WAVES, int RG, int D, int MR>
__global__ __launch_bounds__(WAVES * 64) void gemv_mfma_lds_group_deq_kernel(GemvGroupDeq grp, int m_rows) {
  GemvArgs g;
  DequantParams dq;
  int block;
  pick_member(grp, (int)blockIdx.x, &g, &dq, &block);
  gemv_mfma_lds_body<WAVES, RG, D, MR, 0, true>(g, m_rows, RequantParams{}, dq, block);
}

template <int WAVES, int D, typename F>
static int with_row_class(int m, F &&f) {  // rows rounded up to 2, 4, 8, 16 or 32
  using std::integral_constant;
  if (m <= 2) return f(integral_constant<int, 2>());
  if (m <= 4) return f(integral_constant<int, 4>());
  if (m <= 8) return f(integral_constant<int, 8>());
  if (m <= 16) return f(integral_constant<int, 16>());
  return f(integral_constant<int, 32>());
}

// 33..64 rows: four groups of 16 activation rows against every weight fragment, two steps per pass (the staging
// area of 64 rows and the accumulators leave room for no more).  Measured against the 64 x 64 GEMM tiles these row
// counts ran on before (us per launch at 64 rows): 12288 x 4096 17.9 -> 14.9, 4096 x 4096 15.8 -> 8.9,
// 4096 x 11008 34.9 -> 18.7.
// 65..128 rows against at most 4096 channels with K >= 1024: eight fragments per weight fragment, one channel group
// per workgroup (the staging area of 128 rows takes the LDS of a CU, so more than 4096 channels would need a second
// round of workgroups, and shorter reductions do not pay for the set-up).  Every workgroup re-reads M / 16 = 8
// activation bytes per weight byte from the L2s, which is what bounds it; the GEMM's weight-stream tiles of 64
// channels, the alternative, occupy at most N / 64 CUs (us per launch at 128 rows, weights not cache-resident:
// 4096 x 4096 22.6 -> 14.5, 4096 x 11008 52.7 -> 31.5; with the weights in the caches the two are level at
// 4096 x 4096, 13.3 against 13.5).  Two channel groups per workgroup with one step per pass (what the LDS then has
// room for) were 10-15 % ahead of the tiles between 4096 and 8192 channels and behind them above, and were not kept.
static int launch_mfma_lds_128(const GemvArgs &g, int m, const RequantParams &rq, hipStream_t stream) {
  hipLaunchKernelGGL((gemv_mfma_lds_kernel<8, 1, 2, 128>), dim3((g.n + 15) / 16), dim3(512), 0, stream, g, m, rq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

static int launch_mfma_lds_deq_128(const GemvArgs &g, int m, const DequantParams &dq, hipStream_t stream) {
  hipLaunchKernelGGL((gemv_mfma_lds_deq_kernel<8, 1, 2, 128>), dim3((g.n + 15) / 16), dim3(512), 0, stream, g, m, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int RG>
static int launch_mfma_lds_64(const GemvArgs &g, int m, const RequantParams &rq, hipStream_t stream) {
  const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
  hipLaunchKernelGGL((gemv_mfma_lds_kernel<8, RG, 2, 64>), dim3(blocks), dim3(512), 0, stream, g, m, rq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int RG>
static int launch_mfma_lds_deq_64(const GemvArgs &g, int m, const DequantParams &dq, hipStream_t stream) {
  const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
  hipLaunchKernelGGL((gemv_mfma_lds_deq_kernel<8, RG, 2, 64>), dim3(blocks), dim3(512), 0, stream, g, m, dq);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int WAVES, int RG, int D, typename P>
static int launch_group_mfma_lds(GemvGroupT<P> &grp, int m, hipStream_t stream) {
  int blocks = 0;
  for (int i = 0; i < grp.count; ++i) {
    blocks += (grp.g[i].n + RG * 16 - 1) / (RG * 16);
    grp.block_end[i] = blocks;
  }
  return with_row_class<WAVES, D>(m, [&](auto mr) {
    if constexpr (std::is_same<P, DequantParams>::value) {
      hipLaunchKernelGGL((gemv_mfma_lds_group_deq_kernel<WAVES, RG, D, decltype(mr)::value>), dim3(blocks),
                         dim3(WAVES * 64), 0, stream, grp, m);
    } else {
      hipLaunchKernelGGL((gemv_mfma_lds_group_kernel<WAVES, RG, D, decltype(mr)::value>), dim3(blocks),
                         dim3(WAVES * 64), 0, stream, grp, m);
    }
    MI_HIP_CHECK(hipGetLastError());
    return (int)MI_OK;
  });
}

template <int WAVES, int RG, int D>
static int launch_mfma_lds(const GemvArgs &g, int m, const RequantParams &rq, hipStream_t stream) {
  const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
  return with_row_class<WAVES, D>(m, [&](auto mr) {
    hipLaunchKernelGGL((gemv_mfma_lds_kernel<WAVES, RG, D, decltype(mr)::value>), dim3(blocks), dim3(WAVES * 64), 0,
                       stream, g, m, rq);
    MI_HIP_CHECK(hipGetLastError());
    return (int)MI_OK;
  });
}


__global__ __launch_bounds__(256) void block_weights_kernel(const int8_t *__restrict__ w, int ldw, int kblocks,
                                                            int64_t chunks, int8_t *__restrict__ blocked) {
  // one 16-byte chunk per thread; destination order, so the stores coalesce
  for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * blockDim.x) {
    const int in_block = (int)(c & 63);
    const int64_t blk = c >> 6;
    const int row = (int)(blk / kblocks) * 16 + (in_block & 15);
    const int kbyte = (int)(blk % kblocks) * 64 + (in_block >> 4) * 16;
    *reinterpret_cast<v4i *>(blocked + c * 16) = *reinterpret_cast<const v4i *>(w + (int64_t)row * ldw + kbyte);
  }
}

int launch_block_weights(const int8_t *w, int n_pad, int k_pad, int ldw, int8_t *blocked, hipStream_t stream) {
  const int64_t chunks = (int64_t)n_pad * k_pad / 16;
  const int64_t want = (chunks + 255) / 256;
  hipLaunchKernelGGL(block_weights_kernel, dim3((unsigned)(want > 65536 ? 65536 : want)), dim3(256), 0, stream, w, ldw,
                     k_pad / 64, chunks, blocked);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

template <int WAVES, int RG, int D>
static int launch_mfma_lds_deq(const GemvArgs &g, int m, const DequantParams &dq, hipStream_t stream) {
  const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
  return with_row_class<WAVES, D>(m, [&](auto mr) {
    hipLaunchKernelGGL((gemv_mfma_lds_deq_kernel<WAVES, RG, D, decltype(mr)::value>), dim3(blocks), dim3(WAVES * 64),
                       0, stream, g, m, dq);
    MI_HIP_CHECK(hipGetLastError());
    return (int)MI_OK;
  });
}

// Measurement aid, off unless the environment says MI355X_DIAG_GEMV=1, 2 or 3 when the library is first used: a
// single-matrix launch with 5..8 activation rows then runs a build of the matrix-core kernel without its activation
// fetches (1), without the barrier before the final sum (2) or without both (3).  The results are wrong; the launch
// times show what each of the two costs.
static int gemv_diag() {
  static const int v = [] {
    const char *e = getenv("MI355X_DIAG_GEMV");
    return e != nullptr ? atoi(e) & 3 : 0;
  }();
  return v;
}

template <int RG, int D>
static int launch_mfma_lds_diag(const GemvArgs &g, int m, const RequantParams &rq, hipStream_t stream) {
  const int blocks = (g.n + RG * 16 - 1) / (RG * 16);
  switch (gemv_diag()) {
    case 1: hipLaunchKernelGGL((gemv_mfma_lds_kernel<8, RG, D, 8, 1>), dim3(blocks), dim3(512), 0, stream, g, m, rq); break;
    case 2: hipLaunchKernelGGL((gemv_mfma_lds_kernel<8, RG, D, 8, 2>), dim3(blocks), dim3(512), 0, stream, g, m, rq); break;
    default: hipLaunchKernelGGL((gemv_mfma_lds_kernel<8, RG, D, 8, 3>), dim3(blocks), dim3(512), 0, stream, g, m, rq); break;
  }
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

// Two activation rows run faster on the matrix-core kernel than on the v_dot4 kernel (measured over a decoder layer:
// 4.78 against 4.67 TB/s) when the handle has the blocked weight copy; without it the v_dot4 kernel takes them.
static bool prefers_mfma(int m, const WeightView &wv) {
  return m > kGemvDotRows || (m == 2 && wv.blocked != nullptr);
}

static int check_gemv_operands(const int8_t *a, int64_t lda, int m, int k, const WeightView &wv, int n, const int8_t *c) {
  if (a == nullptr || wv.w == nullptr || c == nullptr) {
    set_error("gemv: null pointer");
    return MI_NULL_PTR;
  }
  if (m < 1 || !gemv_takes_rows(m, n, wv.k_pad) || n <= 0 || k <= 0 || (k & 15) != 0 || (lda & 15) != 0 || lda < k ||
      wv.k_pad % kKPad != 0 || wv.k_pad < k || wv.ldw < wv.k_pad || (wv.ldw & 15) != 0 ||
      (reinterpret_cast<uintptr_t>(a) & 15) != 0 ||
      (int64_t)(m - 1) * lda + k >= (int64_t)1 << 30 || wv.k_pad > 1 << 20 ||  // (32-bit buffer offsets)
      (m <= kGemvDotRows && (int64_t)m * round_up(k, 1024) > 160 * 1024 - 1024)) {
    set_error("gemv: unsupported operand geometry m=%d n=%d k=%d lda=%lld", m, n, k, (long long)lda);
    return MI_PARAM_INVALID;
  }
  if (m > kGemvDotRows && wv.blocked == nullptr) {
    set_error("gemv: the blocked weight copy is missing");
    return MI_NULL_PTR;
  }
  return MI_OK;
}

int launch_gemv_group(const int8_t *a, int64_t lda, int m, int k, int count, const WeightView *wv, const int *n,
                      const RequantParams *rq, int8_t *const *c, hipStream_t stream) {
  if (count < 1 || count > kGemvGroupMax) {
    set_error("gemv group: %d members (1..%d)", count, kGemvGroupMax);
    return MI_PARAM_INVALID;
  }
  if (m > kGemvGroupMaxRows) {
    set_error("gemv group: %d rows (1..%d)", m, kGemvGroupMaxRows);
    return MI_PARAM_INVALID;
  }
  GemvGroup grp{};
  grp.count = count;
  int n_max = 0, k_pad_max = 0;
  bool mfma = true;  // every member has what the matrix-core kernel needs
  for (int i = 0; i < count; ++i) {
    const int rc = check_gemv_operands(a, lda, m, k, wv[i], n[i], c[i]);
    if (rc != MI_OK) return rc;
    mfma = mfma && prefers_mfma(m, wv[i]);
    grp.g[i] = GemvArgs{a, lda, k / 16, wv[i].w, wv[i].ldw, wv[i].k_pad, n[i], c[i], n[i]};
    grp.rq[i] = rq[i];
    n_max = std::max(n_max, n[i]);
    k_pad_max = std::max(k_pad_max, wv[i].k_pad);
  }
  if (mfma) {  // the same choices as for a single matrix, made for the group's largest member
    for (int i = 0; i < count; ++i) grp.g[i].w = wv[i].blocked;
    const bool wide = n_max >= 8192 && k_pad_max <= 4096;
    // (17..32 rows stage twice the rows: four steps per pass keep the staging areas of two workgroups in a CU's LDS)
    if (m > 16) return wide ? launch_group_mfma_lds<8, 2, 4>(grp, m, stream) : launch_group_mfma_lds<8, 1, 4>(grp, m, stream);
    return wide ? launch_group_mfma_lds<8, 2, 4>(grp, m, stream) : launch_group_mfma_lds<8, 1, 8>(grp, m, stream);
  }
  return m == 1 ? launch_group_m<1>(grp, stream) : launch_group_m<2>(grp, stream);
}

int launch_gemv_requant(const int8_t *a, int64_t lda, int m, int k, const WeightView &wv, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream) {
  const int8_t *w = wv.w;
  const int k_pad = wv.k_pad;
  const int rc = check_gemv_operands(a, lda, m, k, wv, n, c);
  if (rc != MI_OK) return rc;
  GemvArgs g{a, lda, k / 16, w, wv.ldw, k_pad, n, c, ldc};
  if (prefers_mfma(m, wv)) {
    g.w = wv.blocked;
    // three 16-channel groups per workgroup (a third of the activation traffic) once there are enough channels to
    // fill the device with 8-wave workgroups and the rows are short enough for a wave's share to be in flight at once
    if (m > 64) return launch_mfma_lds_128(g, m, rq, stream);
    if (m > 32) {
      return n >= 8192 && k_pad <= 4096 ? launch_mfma_lds_64<3>(g, m, rq, stream) : launch_mfma_lds_64<1>(g, m, rq, stream);
    }
    if (gemv_diag() != 0 && m > 4 && m <= 8) {
      return n >= 8192 && k_pad <= 4096 ? launch_mfma_lds_diag<3, 4>(g, m, rq, stream)
                                        : launch_mfma_lds_diag<1, 8>(g, m, rq, stream);
    }
    if (m > 16 && !(n >= 8192 && k_pad <= 4096)) return launch_mfma_lds<8, 1, 4>(g, m, rq, stream);
    if (n >= 8192 && k_pad <= 4096) return launch_mfma_lds<8, 3, 4>(g, m, rq, stream);
    return launch_mfma_lds<8, 1, 8>(g, m, rq, stream);
  }
  return m == 1 ? launch_m<1>(g, rq, stream) : launch_m<2>(g, rq, stream);
}

// The dynamic-quant MatMul at 1..64 rows: the matrix-core decode kernel on the blocked weight copy with the fp32
// epilogue; the same configurations as for the requantising form.
int launch_gemv_dequant(const int8_t *a, int64_t lda, int m, int k, const WeightView &wv, int n,
                        const DequantParams &dq, float *c, int64_t ldc, hipStream_t stream) {
  const int rc = check_gemv_operands(a, lda, m, k, wv, n, reinterpret_cast<const int8_t *>(c));
  if (rc != MI_OK) return rc;
  if (m == 1) {  // one row: the v_dot4 kernel on the row-major weights, as for the requantising MatMul
    const GemvArgs g1{a, lda, k / 16, wv.w, wv.ldw, wv.k_pad, n, reinterpret_cast<int8_t *>(c), ldc};
    return with_config<1>((g1.kchunks + 63) >> 6, [&](auto r, auto d, auto direct, auto ks) {
      return launch_mrdx_deq<1, decltype(r)::value, decltype(d)::value, decltype(direct)::value, decltype(ks)::value>(
          g1, dq, stream);
    });
  }
  if (wv.blocked == nullptr) {
    set_error("gemv: the blocked weight copy is missing");
    return MI_NULL_PTR;
  }
  GemvArgs g{a, lda, k / 16, wv.blocked, wv.ldw, wv.k_pad, n, reinterpret_cast<int8_t *>(c), ldc};
  const bool wide = n >= 8192 && wv.k_pad <= 4096;
  if (m > 64) return launch_mfma_lds_deq_128(g, m, dq, stream);
  if (m > 32) return wide ? launch_mfma_lds_deq_64<3>(g, m, dq, stream) : launch_mfma_lds_deq_64<1>(g, m, dq, stream);
  if (wide) return launch_mfma_lds_deq<8, 3, 4>(g, m, dq, stream);
  return m > 16 ? launch_mfma_lds_deq<8, 1, 4>(g, m, dq, stream) : launch_mfma_lds_deq<8, 1, 8>(g, m, dq, stream);
}

// The dynamic-quant MatMuls that share their input, as one launch (mi_dynmm_run_group): one row on the dot kernel,
// 2..32 rows on the matrix-core kernel (every member then needs its blocked weight copy).
int launch_gemv_group_dequant(const int8_t *a, int64_t lda, int m, int k, int count, const WeightView *wv, const int *n,
                              const DequantParams *dq, float *const *c, hipStream_t stream) {
  if (count < 1 || count > kGemvGroupMax) {
    set_error("gemv group: %d members (1..%d)", count, kGemvGroupMax);
    return MI_PARAM_INVALID;
  }
  if (m > kGemvGroupMaxRows) {
    set_error("gemv group: %d rows (1..%d)", m, kGemvGroupMaxRows);
    return MI_PARAM_INVALID;
  }
  GemvGroupDeq grp{};
  grp.count = count;
  int n_max = 0, k_pad_max = 0;
  for (int i = 0; i < count; ++i) {
    const int rc = check_gemv_operands(a, lda, m, k, wv[i], n[i], reinterpret_cast<const int8_t *>(c[i]));
    if (rc != MI_OK) return rc;
    if (m > 1 && wv[i].blocked == nullptr) {
      set_error("gemv group: the blocked weight copy is missing");
      return MI_NULL_PTR;
    }
    grp.g[i] = GemvArgs{a, lda, k / 16, m == 1 ? wv[i].w : wv[i].blocked, wv[i].ldw, wv[i].k_pad, n[i],
                        reinterpret_cast<int8_t *>(c[i]), n[i]};
    grp.rq[i] = dq[i];
    n_max = std::max(n_max, n[i]);
    k_pad_max = std::max(k_pad_max, wv[i].k_pad);
  }
  if (m == 1) return launch_group_m<1>(grp, stream);
  const bool wide = n_max >= 8192 && k_pad_max <= 4096;
  if (m > 16) return wide ? launch_group_mfma_lds<8, 2, 4>(grp, m, stream) : launch_group_mfma_lds<8, 1, 4>(grp, m, stream);
  return wide ? launch_group_mfma_lds<8, 2, 4>(grp, m, stream) : launch_group_mfma_lds<8, 1, 8>(grp, m, stream);
}

}  // namespace mi
