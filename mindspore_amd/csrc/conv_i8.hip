// Data-movement kernels in front of the GEMM for Conv2D int8, and the depthwise convolution.
//   pad_rows : [rows][k] -> zero-padded [rows][k16]           (activations whose K is not a multiple of 16)
//   im2col   : NHWC image -> [pixels][k16], K order (kh, kw, ic) as Im2ColPackUnitInt8Opt lays rows out
//              (reference mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/conv_int8.c:758-807); taps outside
//              the image take `fill`: the input zero point for the im2col convolution (conv_int8.c:877) and 0 for
//              the strided/padded 1x1 convolution (Conv1x1InputPack into a zeroed buffer,
//              .../nnacl/base/conv1x1_base.c:19-40, mindspore/lite/src/litert/kernel/cpu/int8/
//              convolution_1x1_int8.cc:396)
//   conv_dw  : depthwise conv + requantisation (ConvDwInt8 / ConvDwInt8Post,
//              .../nnacl/int8/conv_depthwise_int8.c:24-140)
//   conv_smallk : dense convolution with kernel_h * kernel_w * in_c <= 64 in one launch, gathered from the image
// The first three are HBM/latency bound byte movers: one thread produces 16 contiguous output bytes (or one output
// element for the depthwise kernel, consecutive threads on consecutive channels) so stores coalesce.
#include "common.h"
#include "quant_math.h"

namespace mi {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void pad_rows_kernel(const int8_t *__restrict__ src, int64_t src_ld, int rows,
                                                       int k, int8_t *__restrict__ dst, int k16) {
  const int chunks_per_row = k16 >> 4;
  const int64_t total = (int64_t)rows * chunks_per_row;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int row = (int)(idx / chunks_per_row), ch = (int)(idx - (int64_t)row * chunks_per_row);
    const int8_t *s = src + (int64_t)row * src_ld + ch * 16;
    union {
      v4i v;
      int8_t b[16];
    } u;
#pragma unroll
    for (int j = 0; j < 16; ++j) u.b[j] = (ch * 16 + j < k) ? s[j] : (int8_t)0;
    *reinterpret_cast<v4i *>(dst + (int64_t)row * k16 + ch * 16) = u.v;
  }
}

int launch_pad_rows(const int8_t *src, int64_t src_ld, int rows, int k, int8_t *dst, int k16, hipStream_t stream) {
  const int64_t total = (int64_t)rows * (k16 >> 4);
  const int blocks = (int)((total + 255) / 256 < 65535 * 16 ? (total + 255) / 256 : 65535 * 16);
  hipLaunchKernelGGL(pad_rows_kernel, dim3(blocks > 0 ? blocks : 1), dim3(256), 0, stream, src, src_ld, rows, k, dst,
                     k16);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

// Compacts rows: dst[row][0..row_bytes) = src[row][0..row_bytes) with different row strides (used when a GEMM wrote
// into a padded scratch output because the caller's row length does not allow vector stores).
__global__ __launch_bounds__(256) void copy_rows_kernel(const char *__restrict__ src, int64_t src_ld, int rows,
                                                        int row_bytes, char *__restrict__ dst, int64_t dst_ld) {
  const int64_t total = (int64_t)rows * row_bytes;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = idx / row_bytes;
    const int col = (int)(idx - row * row_bytes);
    dst[row * dst_ld + col] = src[row * src_ld + col];
  }
}

int launch_copy_rows(const void *src, int64_t src_ld, int rows, int row_bytes, void *dst, int64_t dst_ld,
                     hipStream_t stream) {
  const int64_t total = (int64_t)rows * row_bytes;
  const int64_t want = (total + 255) / 256;
  const int blocks = (int)(want < 1 ? 1 : (want > 262144 ? 262144 : want));
  hipLaunchKernelGGL(copy_rows_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const char *>(src), src_ld, rows,
                     row_bytes, static_cast<char *>(dst), dst_ld);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

__global__ __launch_bounds__(256) void im2col_kernel(const int8_t *__restrict__ in, ConvGeom g, int fill,
                                                     int8_t *__restrict__ dst, int k16) {
  const int kdim = g.kernel_h * g.kernel_w * g.in_c;
  const int chunks_per_row = k16 >> 4;
  const int64_t pixels = (int64_t)g.batch * g.out_h * g.out_w;
  const int64_t total = pixels * chunks_per_row;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t p = idx / chunks_per_row;
    const int ch = (int)(idx - p * chunks_per_row);
    const int b = (int)(p / ((int64_t)g.out_h * g.out_w));
    const int rem = (int)(p - (int64_t)b * g.out_h * g.out_w);
    const int oh = rem / g.out_w, ow = rem - oh * g.out_w;
    const int ih0 = oh * g.stride_h - g.pad_u, iw0 = ow * g.stride_w - g.pad_l;
    const int8_t *img = in + (int64_t)b * g.in_h * g.in_w * g.in_c;
    union {
      v4i v;
      int8_t b[16];
    } u;
    int kk = ch * 16;
    int tap = kk / g.in_c, ic = kk - tap * g.in_c;
    int kh = tap / g.kernel_w, kw = tap - kh * g.kernel_w;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      int8_t val = 0;
      if (kk + j < kdim) {
        const int ih = ih0 + kh * g.dilation_h, iw = iw0 + kw * g.dilation_w;
        const bool inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
        val = inside ? img[((int64_t)ih * g.in_w + iw) * g.in_c + ic] : (int8_t)fill;
      }
      u.b[j] = val;
      if (++ic == g.in_c) {
        ic = 0;
        if (++kw == g.kernel_w) {
          kw = 0;
          ++kh;
        }
      }
    }
    *reinterpret_cast<v4i *>(dst + p * k16 + ch * 16) = u.v;
  }
}

int launch_im2col(const int8_t *in, const ConvGeom &g, int fill, int8_t *dst, int k16, hipStream_t stream) {
  const int64_t total = (int64_t)g.batch * g.out_h * g.out_w * (k16 >> 4);
  const int64_t want = (total + 255) / 256;
  const int blocks = (int)(want < 1 ? 1 : (want > 1048576 ? 1048576 : want));
  hipLaunchKernelGGL(im2col_kernel, dim3(blocks), dim3(256), 0, stream, in, g, fill, dst, k16);
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

// Dense convolution with a short contraction (kernel_h * kernel_w * in_c <= 64, the first layer of an image network:
// 3x3 on 3 channels is K = 27) without an im2col buffer and its extra launch.  One wave produces 32 output pixels x
// all output channels with v_mfma_i32_32x32x32_i8: lane (r, h) gathers bytes [16h, 16h + 16) of every 32-byte K step
// of pixel r straight from the image, in the K order (kh, kw, ic) of Im2ColPackUnitInt8Opt (conv_int8.c:758-807),
// taps outside the image read as `fill` (conv_int8.c:877), bytes past K as 0; the weights come from the packed
// row-major copy (zero filled past K).  Same exact epilogue as the GEMM.
template <int KSTEPS, int OCB>
__global__ __launch_bounds__(256) void conv_smallk_kernel(const int8_t *__restrict__ in, ConvGeom g, int fill,
                                                          int k_true, const int8_t *__restrict__ w, int ldw,
                                                          RequantParams rq, int8_t *__restrict__ out) {
  const int lane = threadIdx.x & 63, r = lane & 31, h = lane >> 5;
  const int64_t first = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 32;
  const int64_t pixels = (int64_t)g.batch * g.out_h * g.out_w;
  if (first >= pixels) return;  // the whole wave
  const bool live = first + r < pixels;
  const int64_t p = live ? first + r : pixels - 1;
  const int b = (int)(p / ((int64_t)g.out_h * g.out_w));
  const int rem = (int)(p - (int64_t)b * g.out_h * g.out_w);
  const int oh = rem / g.out_w, ow = rem - oh * g.out_w;
  const int ih0 = oh * g.stride_h - g.pad_u, iw0 = ow * g.stride_w - g.pad_l;
  const int8_t *img = in + (int64_t)b * g.in_h * g.in_w * g.in_c;

  // The requantisation parameters of the lane's channels, a block of 32 output channels at a time: prm[q][..] are
  // channels 32 * ob + 8 * q + 4 * h .. + 3.  Fetched without a branch on the channel or on the kind of parameters
  // (the arrays are padded to a multiple of 256 channels and all exist) and all sixteen-plus-four at once: the first
  // block's before the gather, so that they arrive behind it.  Fetched where they are used, one group of four
  // channels after the other and behind the branches of the previous group's arithmetic, they were four round trips
  // in a row at the end of a 32-channel stem.
  v4i prm[4][5];
  auto fetch_params = [&](int ob) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int nb = ob * 32 + q * 8 + h * 4;
      prm[q][0] = *reinterpret_cast<const v4i *>(rq.mult + nb);
      prm[q][1] = *reinterpret_cast<const v4i *>(rq.bias2 + nb);
      prm[q][2] = *reinterpret_cast<const v4i *>(rq.rshift + nb);
      prm[q][3] = *reinterpret_cast<const v4i *>(rq.zw + nb);
      prm[q][4] = *reinterpret_cast<const v4i *>(rq.lshift + nb);
    }
  };
  fetch_params(0);

  union Frag {
    v4i v;
    int8_t b[16];
  };
  Frag x[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int k0 = 32 * s + 16 * h;
    int tap = k0 / g.in_c, ic = k0 - tap * g.in_c;
    int kh = tap / g.kernel_w, kw = tap - kh * g.kernel_w;
    // no load is predicated: a byte that is not wanted is fetched from the pixel's image origin and replaced, so
    // that all sixteen loads are in flight together
    int8_t raw[16];
    int other[16];  // -1: take the loaded byte; otherwise the value to use instead
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int ih = ih0 + kh * g.dilation_h, iw = iw0 + kw * g.dilation_w;
      const bool in_k = k0 + i < k_true;
      const bool inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
      const int64_t off = (in_k && inside) ? ((int64_t)ih * g.in_w + iw) * g.in_c + ic : 0;
      raw[i] = img[off];
      other[i] = in_k ? (inside ? -1 : (fill & 0xff)) : 0;
      const bool wrap_c = ic + 1 == g.in_c;
      const bool wrap_w = wrap_c && kw + 1 == g.kernel_w;
      ic = wrap_c ? 0 : ic + 1;
      kw = wrap_w ? 0 : (wrap_c ? kw + 1 : kw);
      kh = wrap_w ? kh + 1 : kh;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) x[s].b[i] = other[i] < 0 ? raw[i] : (int8_t)other[i];
  }

  v16i acc[OCB];
#pragma unroll
  for (int ob = 0; ob < OCB; ++ob)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[ob][e] = 0;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
    for (int ob = 0; ob < OCB; ++ob) {
      const v4i wf = *reinterpret_cast<const v4i *>(w + (int64_t)(ob * 32 + r) * ldw + 32 * s + 16 * h);
      acc[ob] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf, x[s].v, acc[ob], 0, 0, 0);
    }
  int rowsum = 0;
  if (rq.has_zw) {
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      rowsum = __builtin_amdgcn_sdot4(x[s].v.x, 0x01010101, rowsum, false);
      rowsum = __builtin_amdgcn_sdot4(x[s].v.y, 0x01010101, rowsum, false);
      rowsum = __builtin_amdgcn_sdot4(x[s].v.z, 0x01010101, rowsum, false);
      rowsum = __builtin_amdgcn_sdot4(x[s].v.w, 0x01010101, rowsum, false);
    }
    rowsum += __shfl_xor(rowsum, 32);
  }

  // acc[ob][4 * q + e] is output channel 32 * ob + 8 * q + 4 * h + e of pixel r
#pragma unroll
  for (int ob = 0; ob < OCB; ++ob) {
    if (ob > 0) fetch_params(ob);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int nb = ob * 32 + q * 8 + h * 4;
      const v4i mult4 = prm[q][0], bias4 = prm[q][1], e4 = prm[q][2], zw4 = prm[q][3], ls4 = prm[q][4];
      union {
        uint32_t u;
        int8_t b[4];
      } o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t v = (uint32_t)acc[ob][q * 4 + e];
        if (rq.has_zw) v -= (uint32_t)rowsum * (uint32_t)zw4[e];
        v += (uint32_t)bias4[e];
        int32_t t;
        if (rq.fast) {
          t = rdiv_pot_fast(srdhm_nosat((int32_t)v, mult4[e]), e4[e], (1 << e4[e]) >> 1);
        } else {
          t = rdiv_pot(srdhm((int32_t)(v << ls4[e]), mult4[e]), e4[e]);
        }
        t = (int32_t)((uint32_t)t + (uint32_t)rq.zo);
        t = t < rq.amax ? t : rq.amax;
        t = t > rq.amin ? t : rq.amin;
        o.b[e] = (int8_t)t;
      }
      if (live && nb < g.out_c) *reinterpret_cast<uint32_t *>(out + p * g.out_c + nb) = o.u;
    }
  }
}

int launch_conv_smallk(const int8_t *in, const ConvGeom &g, int fill, int k_true, const int8_t *w, int ldw,
                       const RequantParams &rq, int8_t *out, hipStream_t stream) {
  const int64_t pixels = (int64_t)g.batch * g.out_h * g.out_w;
  if (k_true < 1 || k_true > 64 || g.out_c < 4 || g.out_c > 128 || (g.out_c & 3) != 0 ||
      (reinterpret_cast<uintptr_t>(out) & 3) != 0 || (reinterpret_cast<uintptr_t>(w) & 15) != 0 || (ldw & 15) != 0 ||
      ldw < 64 || pixels < 1) {
    set_error("conv_smallk: unsupported geometry k=%d oc=%d", k_true, g.out_c);
    return MI_PARAM_INVALID;
  }
  const int64_t waves = (pixels + 31) / 32;
  const int blocks = (int)((waves + 3) / 4);
  const int ocb = (g.out_c + 31) / 32, ksteps = (k_true + 31) / 32;
#define MI_SMALLK(KS, OB)                                                                                       \
  hipLaunchKernelGGL((conv_smallk_kernel<KS, OB>), dim3(blocks), dim3(256), 0, stream, in, g, fill, k_true, w, ldw, \
                     rq, out)
  if (ksteps == 1) {
    if (ocb == 1) MI_SMALLK(1, 1);
    else if (ocb == 2) MI_SMALLK(1, 2);
    else if (ocb == 3) MI_SMALLK(1, 3);
    else MI_SMALLK(1, 4);
  } else {
    if (ocb == 1) MI_SMALLK(2, 1);
    else if (ocb == 2) MI_SMALLK(2, 2);
    else if (ocb == 3) MI_SMALLK(2, 3);
    else MI_SMALLK(2, 4);
  }
#undef MI_SMALLK
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

__global__ __launch_bounds__(256) void conv_dw_kernel(const int8_t *__restrict__ in, ConvGeom g,
                                                      const int16_t *__restrict__ w16,
                                                      const int32_t *__restrict__ bias, int zx8, RequantParams rq,
                                                      int8_t *__restrict__ out) {
  const int ch = g.out_c;
  const int64_t total = (int64_t)g.batch * g.out_h * g.out_w * ch;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t p = idx / ch;
    const int c = (int)(idx - p * ch);
    const int b = (int)(p / ((int64_t)g.out_h * g.out_w));
    const int rem = (int)(p - (int64_t)b * g.out_h * g.out_w);
    const int oh = rem / g.out_w, ow = rem - oh * g.out_w;
    const int8_t *img = in + (int64_t)b * g.in_h * g.in_w * ch;
    uint32_t acc = (uint32_t)bias[c];
    for (int kh = 0; kh < g.kernel_h; ++kh) {
      const int ih = oh * g.stride_h - g.pad_u + kh * g.dilation_h;
      if (ih < 0 || ih >= g.in_h) continue;
      for (int kw = 0; kw < g.kernel_w; ++kw) {
        const int iw = ow * g.stride_w - g.pad_l + kw * g.dilation_w;
        if (iw < 0 || iw >= g.in_w) continue;
        const int16_t xv = (int16_t)((int)img[((int64_t)ih * g.in_w + iw) * ch + c] - zx8);
        const int16_t wv = w16[(kh * g.kernel_w + kw) * ch + c];
        acc += (uint32_t)((int32_t)xv * (int32_t)wv);
      }
    }
    const int32_t mult = rq.mult[c], e = rq.rshift[c], ls = rq.lshift[c];
    int32_t y = rdiv_pot(srdhm((int32_t)(acc << ls), mult), e);
    y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
    y = y > rq.amin ? y : rq.amin;  // MSMAX first, then MSMIN (conv_depthwise_int8.c:49-50)
    y = y < rq.amax ? y : rq.amax;
    out[idx] = (int8_t)y;
  }
}

// Channel-vectorised variant for C % 8 == 0: one thread produces CG = 16 (or 8, when C is not a multiple of 16)
// consecutive channels of one output pixel, so every tap is one CG-byte activation load and 2 * CG bytes of weights,
// and the store is one CG-byte row segment.
// A tap outside the image reads as the input zero point (the matching -zx * w is already in bias_folded), so the
// inner product is sum_t x_t * w_t with no subtraction.  TAPS > 0 (kernel_h * kernel_w known at compile time): the
// loads of all taps are issued before the first multiply.  TAPS == 0: any kernel size, five taps per batch of loads.  FAST: the host
// proved the cheap rounding form exact for every channel (no left shifts to fetch).
template <int TAPS, int CG, bool FAST>
__global__ __launch_bounds__(256) void conv_dw16_kernel(const int8_t *__restrict__ in, ConvGeom g,
                                                        const int16_t *__restrict__ w16,
                                                        const int32_t *__restrict__ bias_folded, int zx8,
                                                        RequantParams rq, int8_t *__restrict__ out) {
  static_assert(CG == 8 || CG == 16, "channels per thread");
  constexpr int XW = CG / 4;  // dwords of activations per tap
  constexpr int WQ = CG / 8;  // 16-byte vectors of int16 weights per tap
  const int ch = g.out_c, groups = ch / CG;
  const int64_t total = (int64_t)g.batch * g.out_h * g.out_w * groups;
  const int zsplat = (zx8 & 0xff) * 0x01010101;
  union XV {
    int32_t d[XW];
    int8_t b[CG];
  };
  union WV {
    v4i v[WQ];
    int16_t h[CG];
  };
  auto load_x = [](const int8_t *p, XV *x) {
    if constexpr (CG == 16) {
      const v4i v = *reinterpret_cast<const v4i *>(p);
      x->d[0] = v.x, x->d[1] = v.y, x->d[2] = v.z, x->d[3] = v.w;
    } else {
      const v2i v = *reinterpret_cast<const v2i *>(p);
      x->d[0] = v.x, x->d[1] = v.y;
    }
  };
  // Consecutive workgroup ids are dealt round-robin over the 8 XCDs, each with an L2 of its own; a 3x3 window reads
  // three image rows, so with ids in pixel order every XCD would fetch nearly the whole image (measured: 8.0 MB for
  // a 2.4 MB image).  Ids that share an XCD are mapped to one contiguous band of the output instead.
  int64_t bid = blockIdx.x;
  {
    const int64_t per = gridDim.x >> 3;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  for (int64_t idx = bid * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t p = idx / groups;
    const int c0 = (int)(idx - p * groups) * CG;
    const int b = (int)(p / ((int64_t)g.out_h * g.out_w));
    const int rem = (int)(p - (int64_t)b * g.out_h * g.out_w);
    const int oh = rem / g.out_w, ow = rem - oh * g.out_w;
    const int8_t *img = in + (int64_t)b * g.in_h * g.in_w * ch + c0;
    uint32_t acc[CG];
    {
      const v4i *bp = reinterpret_cast<const v4i *>(bias_folded + c0);
#pragma unroll
      for (int q = 0; q < CG / 4; ++q) {
        const v4i bv = bp[q];
        acc[4 * q + 0] = (uint32_t)bv.x;
        acc[4 * q + 1] = (uint32_t)bv.y;
        acc[4 * q + 2] = (uint32_t)bv.z;
        acc[4 * q + 3] = (uint32_t)bv.w;
      }
    }
    auto mac = [&](XV xv, const WV &wv, bool inside) {
#pragma unroll
      for (int q = 0; q < XW; ++q) xv.d[q] = inside ? xv.d[q] : zsplat;
#pragma unroll
      for (int j = 0; j < CG; ++j) acc[j] += (uint32_t)((int32_t)xv.b[j] * (int32_t)wv.h[j]);  // 8 bit x 10 bit
    };
    auto tap_address = [&](int kh, int kw, bool *inside) -> const int8_t * {
      const int ih = oh * g.stride_h - g.pad_u + kh * g.dilation_h;
      const int iw = ow * g.stride_w - g.pad_l + kw * g.dilation_w;
      *inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
      const int ihc = ih < 0 ? 0 : (ih >= g.in_h ? g.in_h - 1 : ih);
      const int iwc = iw < 0 ? 0 : (iw >= g.in_w ? g.in_w - 1 : iw);
      return img + ((int64_t)ihc * g.in_w + iwc) * ch;
    };
    if (TAPS > 0) {
      XV xv[TAPS > 0 ? TAPS : 1];
      WV wv[TAPS > 0 ? TAPS : 1];
      bool inside[TAPS > 0 ? TAPS : 1];
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const int kh = t / g.kernel_w, kw = t - kh * g.kernel_w;
        load_x(tap_address(kh, kw, &inside[t]), &xv[t]);
        const v4i *wp = reinterpret_cast<const v4i *>(w16 + (int64_t)t * ch + c0);
#pragma unroll
        for (int q = 0; q < WQ; ++q) wv[t].v[q] = wp[q];
      }
#pragma unroll
      for (int t = 0; t < TAPS; ++t) mac(xv[t], wv[t], inside[t]);
    } else {
      // five taps at a time (a row of a 5x5 kernel): their loads are issued together, so a kernel of T taps costs
      // T / 5 memory round trips instead of T
      constexpr int B = 5;
      const int taps = g.kernel_h * g.kernel_w;
      int kh = 0, kw = 0;  // of tap t0 + u, kept by stepping (no division per tap)
      for (int t0 = 0; t0 < taps; t0 += B) {
        XV xv[B];
        WV wv[B];
        bool inside[B];
#pragma unroll
        for (int u = 0; u < B; ++u) {
          const bool past = t0 + u >= taps;  // past the last tap: a re-read of the last one that is not used
          const int t = past ? taps - 1 : t0 + u;
          load_x(tap_address(past ? g.kernel_h - 1 : kh, past ? g.kernel_w - 1 : kw, &inside[u]), &xv[u]);
          const bool wrap_w = kw + 1 == g.kernel_w;
          kw = wrap_w ? 0 : kw + 1;
          kh = wrap_w ? kh + 1 : kh;
          const v4i *wp = reinterpret_cast<const v4i *>(w16 + (int64_t)t * ch + c0);
#pragma unroll
          for (int q = 0; q < WQ; ++q) wv[u].v[q] = wp[q];
        }
#pragma unroll
        for (int u = 0; u < B; ++u)
          if (t0 + u < taps) mac(xv[u], wv[u], inside[u]);
      }
    }
    union {
      int32_t d[XW];
      int8_t b[CG];
    } o;
#pragma unroll
    for (int q = 0; q < CG / 4; ++q) {
      const v4i m4 = *reinterpret_cast<const v4i *>(rq.mult + c0 + 4 * q);
      const v4i rs4 = *reinterpret_cast<const v4i *>(rq.rshift + c0 + 4 * q);
      v4i ls4 = {0, 0, 0, 0};
      if (!FAST) ls4 = *reinterpret_cast<const v4i *>(rq.lshift + c0 + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        int32_t y;
        if (FAST) {
          y = rdiv_pot_fast(srdhm_nosat((int32_t)acc[4 * q + e], m4[e]), rs4[e], (1 << rs4[e]) >> 1);
        } else {
          y = rdiv_pot(srdhm((int32_t)(acc[4 * q + e] << ls4[e]), m4[e]), rs4[e]);
        }
        y = (int32_t)((uint32_t)y + (uint32_t)rq.zo);
        y = y > rq.amin ? y : rq.amin;  // MSMAX first, then MSMIN (conv_depthwise_int8.c:49-50)
        y = y < rq.amax ? y : rq.amax;
        o.b[4 * q + e] = (int8_t)y;
      }
    }
    if constexpr (CG == 16) {
      *reinterpret_cast<v4i *>(out + p * ch + c0) = v4i{o.d[0], o.d[1], o.d[2], o.d[3]};
    } else {
      *reinterpret_cast<v2i *>(out + p * ch + c0) = v2i{o.d[0], o.d[1]};
    }
  }
}

template <int TAPS, int CG>
static void launch_dw_vec(const int8_t *in, const ConvGeom &g, const int16_t *w16, const int32_t *bias_folded, int zx8,
                          const RequantParams &rq, int8_t *out, hipStream_t stream) {
  const int64_t total = (int64_t)g.batch * g.out_h * g.out_w * (g.out_c / CG);
  const int64_t want = (total + 255) / 256;
  const int blocks = (int)(want < 1 ? 1 : (want > 1048576 ? 1048576 : want));
  if (rq.fast) {
    hipLaunchKernelGGL((conv_dw16_kernel<TAPS, CG, true>), dim3(blocks), dim3(256), 0, stream, in, g, w16, bias_folded,
                       zx8, rq, out);
  } else {
    hipLaunchKernelGGL((conv_dw16_kernel<TAPS, CG, false>), dim3(blocks), dim3(256), 0, stream, in, g, w16, bias_folded,
                       zx8, rq, out);
  }
}

int launch_conv_dw(const int8_t *in, const ConvGeom &g, const int16_t *w16, const int32_t *bias,
                   const int32_t *bias_folded, int zx8, const RequantParams &rq, int8_t *out, hipStream_t stream) {
  const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  const bool vec16 = aligned && (g.out_c & 15) == 0, vec8 = aligned && (g.out_c & 7) == 0;
  const bool taps9 = g.kernel_h * g.kernel_w == 9;
  // kernels larger than 3x3 on few pixels: a thread's chain of taps is what the launch lasts, and there are SIMDs to
  // spare, so half the channels per thread
  const bool k5 = g.kernel_h == 5 && g.kernel_w == 5;  // (compile-time taps: 6.4 instead of 7.2 us)
  const bool long_chain = !taps9 && (int64_t)g.batch * g.out_h * g.out_w * (g.out_c >> 4) < 65536;
  if (vec8 && (!vec16 || long_chain)) {  // 8, 24, 40, ... channels
    if (taps9) launch_dw_vec<9, 8>(in, g, w16, bias_folded, zx8, rq, out, stream);
    else if (k5) launch_dw_vec<25, 8>(in, g, w16, bias_folded, zx8, rq, out, stream);
    else launch_dw_vec<0, 8>(in, g, w16, bias_folded, zx8, rq, out, stream);
  } else if (vec16) {
    if (taps9) launch_dw_vec<9, 16>(in, g, w16, bias_folded, zx8, rq, out, stream);
    else launch_dw_vec<0, 16>(in, g, w16, bias_folded, zx8, rq, out, stream);
  } else {
    const int64_t total = (int64_t)g.batch * g.out_h * g.out_w * g.out_c;
    const int64_t want = (total + 255) / 256;
    const int blocks = (int)(want < 1 ? 1 : (want > 1048576 ? 1048576 : want));
    hipLaunchKernelGGL(conv_dw_kernel, dim3(blocks), dim3(256), 0, stream, in, g, w16, bias, zx8, rq, out);
  }
  MI_HIP_CHECK(hipGetLastError());
  return MI_OK;
}

}  // namespace mi
