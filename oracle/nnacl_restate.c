/*
 * TEST INFRASTRUCTURE ONLY -- see nnacl_restate.h.  CPU restatement of MindSpore Lite's int8 hot path.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   fixed point / multiplier derivation : exact big-integer / rational closed forms + the compiled nnacl
 *   matmul / conv / depthwise           : int64 NumPy evaluation of sum (x-zx)(w-zw) on small shapes,
 *                                         committed golden vectors produced by the compiled nnacl,
 *                                         and live comparison against the compiled nnacl where it is built
 *   dynamic quant / dynamic matmul      : NumPy float32 closed forms + compiled nnacl + golden vectors
 */
#include "nnacl_restate.h"

#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }

/* wrapping int32 helpers: the reference relies on two's-complement wrap of int arithmetic */
static inline int32_t wadd(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
static inline int32_t wsub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
static inline int32_t wmul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }

/* NN/int8/fixed_point.c:26-35.  The sign-dependent nudge followed by a truncating division by 2^31 is
 * floor((a*b + 2^30) / 2^31): ties go toward +infinity.  Only a == b == INT32_MIN saturates. */
int32_t orc_srdhm(int32_t a, int32_t b) {
  if (a == INT32_MIN && b == INT32_MIN) return INT32_MAX;
  int64_t p = (int64_t)a * (int64_t)b + ((int64_t)1 << 30);
  /* floor division by 2^31 without relying on the sign behaviour of >> */
  int64_t q = p / ((int64_t)1 << 31);
  if ((p % ((int64_t)1 << 31)) < 0) q -= 1;
  return (int32_t)q;
}

/* NN/int8/fixed_point.c:48-56.  x / 2^e rounded to nearest, ties away from zero; e is capped at 31. */
int32_t orc_rdiv_pot(int32_t x, int32_t exponent) {
  if (exponent > 31) exponent = 31;
  if (exponent <= 0) return x; /* mask == 0: remainder 0 is never > threshold >= 0 */
  int64_t d = (int64_t)1 << exponent;
  int64_t mag = x < 0 ? -(int64_t)x : (int64_t)x;
  int64_t q = (mag + (d >> 1)) / d; /* round half up on the magnitude == half away from zero */
  return (int32_t)(x < 0 ? -q : q);
}

/* NN/int8/fixed_point.c:66-68.  The pre-multiplication by 2^ls wraps in int32. */
int32_t orc_mul_by_quant_mult(int32_t v, int32_t mult, int32_t ls, int32_t rs) {
  int32_t shifted = wmul(v, (int32_t)((uint32_t)1 << ls));
  return orc_rdiv_pot(orc_srdhm(shifted, mult), -rs);
}

/* NN/int8/quantize.c:113-161.  |m| = q * 2^shift with q in [0.5, 1); mult = q * 2^31 rounded half-up to an
 * integer in [2^30, 2^31); a carry to 2^31 renormalises.  The sign moves onto mult. */
void orc_quantize_multiplier(double m, int32_t *mult, int32_t *shift) {
  if (m == 0.0) { /* +0 and -0 */
    *mult = 0;
    *shift = 0;
    return;
  }
  if (isnan(m)) {
    *mult = 0;
    *shift = 0;
    return;
  }
  if (isinf(m)) {
    *mult = m < 0 ? INT32_MIN : INT32_MAX;
    *shift = 0;
    return;
  }
  int e = 0;
  double q = frexp(fabs(m), &e);            /* exact, handles subnormals */
  uint64_t sig = (uint64_t)ldexp(q, 53);    /* 53-bit significand as an integer in [2^52, 2^53) */
  uint64_t r = ((sig >> 21) + 1u) >> 1;     /* keep 31 bits, round half up */
  if (r == ((uint64_t)1 << 31)) {
    r >>= 1;
    e += 1;
  }
  *shift = e;
  *mult = m < 0 ? -(int32_t)r : (int32_t)r;
}

/* NN/int8/quantize.c:39-51 */
void orc_round_param(double m, int32_t *mult, int32_t *ls, int32_t *rs) {
  int32_t shift = 0;
  orc_quantize_multiplier(m, mult, &shift);
  if (shift < 0) {
    *ls = 0;
    *rs = shift;
  } else {
    *ls = shift;
    *rs = 0;
  }
}

/* NN/int8/quantize.c:76 -- float divide, float add of the converted zero point, round half away, to int32 */
static int32_t quantize_to_int8_unclamped(float real, float scale, int32_t zp) {
  float t = real / scale;
  t = t + (float)zp;
  return (int32_t)round((double)t);
}

/* NN/int8/quantize.c:78-94 */
void orc_act_range(int relu, int relu6, int32_t zp, float scale, int32_t *mn, int32_t *mx) {
  int32_t lo = INT8_MIN, hi = INT8_MAX;
  int32_t q0 = quantize_to_int8_unclamped(0.0f, scale, zp);
  int32_t q6 = quantize_to_int8_unclamped(6.0f, scale, zp);
  if (relu) {
    if (q0 > lo) lo = q0;
  } else if (relu6) {
    if (q0 > lo) lo = q0;
    if (q6 < hi) hi = q6;
  }
  *mn = lo;
  *mx = hi;
}

/* LK/int8/matmul_base_int8.cc:235-273, LK/base/convolution_base.cc:416-427: every tensor scale (double on the
 * lite tensor) is first narrowed to float (QuantArg.scale_, NN/op_base.h:678-681); the product is formed in
 * float, widened, and divided by the widened float output scale. */
void orc_requant_params(double sx, const double *sw, int nfilt, double so, int32_t *mult, int32_t *ls, int32_t *rs) {
  float fx = (float)sx, fo = (float)so;
  for (int i = 0; i < nfilt; ++i) {
    float fw = (float)sw[i];
    volatile float prod = fx * fw; /* volatile: forbid widening/contracting the float product */
    double real = (double)prod / (double)fo;
    orc_round_param(real, &mult[i], &ls[i], &rs[i]);
  }
}

/* NN/int8/quantize.c:53-72.  The reference converts the double VALUE (not its bit pattern) to uint32, so every
 * multiplier below 1 yields (0x40000000, 0, -126); kept as it is.  Domain: 0 <= m < 2^32. */
void orc_round_param_single(double m, int32_t *mult, int32_t *ls, int32_t *rs) {
  const uint32_t bits = (uint32_t)m;
  *mult = (int32_t)(((bits & 0x007FFFFFu) | 0x00800000u) << 7);
  int32_t shift = 127 + 31 - 32 - (int32_t)(bits >> 23);
  shift = -shift;
  if (shift < 0) {
    *ls = 0;
    *rs = shift;
  } else {
    *ls = shift;
    *rs = 0;
  }
}

static int32_t requant_to_i8(int32_t v, int32_t mult, int32_t ls, int32_t rs, int32_t zo, int32_t amin, int32_t amax) {
  int32_t y = wadd(orc_mul_by_quant_mult(v, mult, ls, rs), zo);
  if (y > amax) y = amax; /* MSMIN(maxi, value) first, then MSMAX(mini, value): NN/int8/matmul_int8.c:325-326 */
  if (y < amin) y = amin;
  return y;
}

typedef struct requant_ctx {
  int peroc;
  int32_t *mult, *ls, *rs;
  int32_t amin, amax, zo;
} requant_ctx;

static int requant_ctx_init(requant_ctx *q, double sx, const double *sw, int nfilt, double so, int zo, int act_type) {
  q->peroc = nfilt > 1;
  q->mult = (int32_t *)malloc(sizeof(int32_t) * (size_t)nfilt);
  q->ls = (int32_t *)malloc(sizeof(int32_t) * (size_t)nfilt);
  q->rs = (int32_t *)malloc(sizeof(int32_t) * (size_t)nfilt);
  if (!q->mult || !q->ls || !q->rs) return -1;
  orc_requant_params(sx, sw, nfilt, so, q->mult, q->ls, q->rs);
  orc_act_range(act_type == ORC_ACT_RELU, act_type == ORC_ACT_RELU6, zo, (float)so, &q->amin, &q->amax);
  q->zo = zo;
  return 0;
}

static void requant_ctx_free(requant_ctx *q) {
  free(q->mult);
  free(q->ls);
  free(q->rs);
}

/* Full-quant MatMul / FullConnection.
 *   weights+bias fold  : CalcWeightBiasSums NN/int8/matmul_int8.c:802-819 (called from TransferB,
 *                        LK/int8/matmul_base_int8.cc:360-384)
 *   input row sums     : CalcInputSums NN/int8/matmul_int8.c:786-799 (per-tensor: times zw[0]; per-channel: times 1)
 *   contraction+requant: MatmulInt8Opt NN/int8/matmul_int8.c:296-331
 * b_transpose != 0: W is [N,K] (FullConnection always, LK/int8/fullconnection_int8.cc:33-34); else W is [K,N]. */
int orc_matmul_int8(const int8_t *a, const int8_t *w, const int32_t *bias, int8_t *c, int m, int n, int k,
                    int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so,
                    int zo, int act_type) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != n)) return -1;
  requant_ctx q;
  if (requant_ctx_init(&q, sx, sw, nfilt, so, zo, act_type) != 0) return -1;
  int8_t *wt = NULL; /* [N][K] view */
  const int8_t *wnk = w;
  if (!b_transpose) {
    wt = (int8_t *)malloc((size_t)n * (size_t)k + 1);
    if (!wt) return -1;
    for (int kk = 0; kk < k; ++kk)
      for (int cc = 0; cc < n; ++cc) wt[(size_t)cc * k + kk] = w[(size_t)kk * n + cc];
    wnk = wt;
  }
  int32_t *wb = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
  int32_t *asum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(m > 0 ? m : 1));
  if (!wb || !asum) return -1;
  for (int cc = 0; cc < n; ++cc) {
    int32_t s = 0;
    for (int kk = 0; kk < k; ++kk) s += wnk[(size_t)cc * k + kk];
    int32_t z = q.peroc ? zw[cc] : zw[0];
    int32_t v = wsub(wmul(wmul(k, zx), z), wmul(zx, s));
    if (bias) v = wadd(v, bias[cc]);
    wb[cc] = v;
  }
  for (int r = 0; r < m; ++r) {
    int32_t s = 0;
    for (int kk = 0; kk < k; ++kk) s += a[(size_t)r * k + kk];
    asum[r] = wmul(s, q.peroc ? 1 : zw[0]);
  }
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int r = 0; r < m; ++r) {
    const int8_t *ar = a + (size_t)r * k;
    for (int cc = 0; cc < n; ++cc) {
      const int8_t *wr = wnk + (size_t)cc * k;
      int32_t acc = 0;
      for (int kk = 0; kk < k; ++kk) acc += (int32_t)ar[kk] * (int32_t)wr[kk];
      int32_t isum = q.peroc ? wmul(asum[r], zw[cc]) : asum[r];
      int32_t v = wadd(wsub(acc, isum), wb[cc]);
      int qi = q.peroc ? cc : 0;
      c[(size_t)r * n + cc] = (int8_t)requant_to_i8(v, q.mult[qi], q.ls[qi], q.rs[qi], q.zo, q.amin, q.amax);
    }
  }
  free(wb);
  free(asum);
  free(wt);
  requant_ctx_free(&q);
  return 0;
}

/* Conv2D int8, group == 1.
 * kernel 1x1 -> Convolution1x1Int8CPUKernel (selection LK/int8/convolution_int8_creator.cc:93-94): when stride or
 *   pad is non-trivial the input pixels are gathered into a buffer that was cleared to 0, NOT to the input zero
 *   point (LK/int8/convolution_1x1_int8.cc:359-397,435-444; NN/base/conv1x1_base.c:19-40), so an out-of-image tap
 *   contributes (0 - zx) * (w - zw).  Bias fold: InitBiasByzp :158-176.
 * otherwise -> ConvolutionInt8CPUKernel: im2col rows are pre-filled with zx (NN/int8/conv_int8.c:877) so an
 *   out-of-image tap contributes nothing; K order is (kh, kw, ic) (:794,802); bias fold
 *   LK/int8/convolution_int8.cc:131-142.
 * 3x3 stride 1 dilation 1: the reference's choice depends on the CPU (LK/int8/convolution_int8_creator.cc:81-94).
 *   ARM64 cores with the dot-product extension run ConvolutionInt8CPUKernel as above, and that is what this function
 *   computes; every other build (x86 included) runs an integer Winograd kernel, which is NOT restated here (the
 *   product declines those convolutions unless asked for the exact form). */
int orc_conv_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const orc_conv_shape *s,
                  double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo, int act_type) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != s->out_c)) return -1;
  requant_ctx q;
  if (requant_ctx_init(&q, sx, sw, nfilt, so, zo, act_type) != 0) return -1;
  const int is_1x1 = (s->kernel_h == 1 && s->kernel_w == 1);
  const int32_t oob_value = is_1x1 ? 0 : zx;
  const int kdim = s->kernel_h * s->kernel_w * s->in_c;
  const int64_t opix = (int64_t)s->batch * s->out_h * s->out_w;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t p = 0; p < opix; ++p) {
    int b = (int)(p / ((int64_t)s->out_h * s->out_w));
    int rem = (int)(p % ((int64_t)s->out_h * s->out_w));
    int oh = rem / s->out_w, ow = rem % s->out_w;
    const int8_t *inb = in + (size_t)b * s->in_h * s->in_w * s->in_c;
    for (int oc = 0; oc < s->out_c; ++oc) {
      const int32_t z = q.peroc ? zw[oc] : zw[0];
      const int8_t *wr = w + (size_t)oc * kdim;
      int32_t acc = bias ? bias[oc] : 0;
      for (int kh = 0; kh < s->kernel_h; ++kh) {
        int ih = oh * s->stride_h - s->pad_u + kh * s->dilation_h;
        for (int kw = 0; kw < s->kernel_w; ++kw) {
          int iw = ow * s->stride_w - s->pad_l + kw * s->dilation_w;
          int inside = ih >= 0 && ih < s->in_h && iw >= 0 && iw < s->in_w;
          const int8_t *px = inside ? inb + ((size_t)ih * s->in_w + iw) * s->in_c : NULL;
          const int8_t *wt = wr + (size_t)(kh * s->kernel_w + kw) * s->in_c;
          for (int ic = 0; ic < s->in_c; ++ic) {
            int32_t x = inside ? (int32_t)px[ic] : oob_value;
            acc = wadd(acc, wmul(wsub(x, zx), wsub((int32_t)wt[ic], z)));
          }
        }
      }
      int qi = q.peroc ? oc : 0;
      out[(size_t)p * s->out_c + oc] = (int8_t)requant_to_i8(acc, q.mult[qi], q.ls[qi], q.rs[qi], q.zo, q.amin, q.amax);
    }
  }
  requant_ctx_free(&q);
  return 0;
}

/* Depthwise conv int8 with per-tensor activations.
 * Weights are pre-offset by their zero point into int16 (LK/int8/convolution_depthwise_int8.cc:61-89, weight
 * memory [C][KH*KW]); the input zero point is narrowed to int8 before the subtraction
 * (NN/int8/conv_depthwise_int8.c:24-33, parameter `int8_t input_zp`) and the difference to int16; taps outside the
 * image are skipped (:107-131); requantisation ConvDwInt8Post :36-78. */
int orc_conv_dw_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const orc_conv_shape *s,
                     double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo,
                     int act_type) {
  const int ch = s->out_c;
  if (s->in_c != ch || nfilt < 1 || (nfilt > 1 && nfilt != ch)) return -1;
  requant_ctx q;
  if (requant_ctx_init(&q, sx, sw, nfilt, so, zo, act_type) != 0) return -1;
  const int8_t zx8 = (int8_t)zx;
  const int kplane = s->kernel_h * s->kernel_w;
  const int64_t opix = (int64_t)s->batch * s->out_h * s->out_w;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t p = 0; p < opix; ++p) {
    int b = (int)(p / ((int64_t)s->out_h * s->out_w));
    int rem = (int)(p % ((int64_t)s->out_h * s->out_w));
    int oh = rem / s->out_w, ow = rem % s->out_w;
    const int8_t *inb = in + (size_t)b * s->in_h * s->in_w * ch;
    for (int c = 0; c < ch; ++c) {
      const int32_t z = q.peroc ? zw[c] : zw[0];
      int32_t acc = bias ? bias[c] : 0;
      for (int kh = 0; kh < s->kernel_h; ++kh) {
        int ih = oh * s->stride_h - s->pad_u + kh * s->dilation_h;
        if (ih < 0 || ih >= s->in_h) continue;
        for (int kw = 0; kw < s->kernel_w; ++kw) {
          int iw = ow * s->stride_w - s->pad_l + kw * s->dilation_w;
          if (iw < 0 || iw >= s->in_w) continue;
          int16_t xv = (int16_t)((int32_t)inb[((size_t)ih * s->in_w + iw) * ch + c] - (int32_t)zx8);
          int16_t wv = (int16_t)((int32_t)w[(size_t)c * kplane + kh * s->kernel_w + kw] - z);
          acc = wadd(acc, (int32_t)xv * (int32_t)wv);
        }
      }
      int qi = q.peroc ? c : 0;
      /* ConvDwInt8Post clamps MSMAX(value, acc_min) first, then MSMIN(value, acc_max):
       * NN/int8/conv_depthwise_int8.c:49-52 (the other order than MatmulInt8Opt; differs only if amin > amax) */
      int32_t y = wadd(orc_mul_by_quant_mult(acc, q.mult[qi], q.ls[qi], q.rs[qi]), q.zo);
      if (y < q.amin) y = q.amin;
      if (y > q.amax) y = q.amax;
      out[(size_t)p * ch + c] = (int8_t)y;
    }
  }
  requant_ctx_free(&q);
  return 0;
}

/* NN/int8/dynamic_quant_int8.c:19-27: strict < and > updates, so a NaN is never selected.  The Lite wrapper scans
 * in up to 8 buckets and merges them with the same comparisons (LK/int8/dynamic_quant.cc:118-163); min and max are
 * order-independent, so one scan gives the same pair. */
void orc_minmax_fp32(const float *x, int64_t n, float *mn, float *mx) {
  float lo = *mn, hi = *mx;
  for (int64_t i = 0; i < n; ++i) {
    float v = x[i];
    if (v < lo) lo = v;
    if (v > hi) hi = v;
  }
  *mn = lo;
  *mx = hi;
}

/* LK/int8/dynamic_quant.cc:156-186.  Asymmetric: float range, float division by 255, widened to double; the zero
 * point is computed in double.  Symmetric: 2*max(|max|,|min|)/254 in float, zero point 0. */
void orc_dynquant_params(float mn, float mx, int symmetric, double *scale, int32_t *zp) {
  if (!symmetric) {
    volatile float range = mx - mn;
    if (range <= 0) range = 0.01f;
    volatile float sf = range / 255.0f;
    double sc = (double)sf;
    *scale = sc;
    *zp = (int32_t)round(-128.0 - (double)mn / sc);
  } else {
    float a = fabsf(mx), b = fabsf(mn);
    float big = (a < b) ? b : a; /* std::max(a, b) returns a unless a < b */
    volatile float two = 2.0f * big;
    volatile float sf = two / 254.0f;
    *scale = (double)sf;
    *zp = 0;
  }
}

/* NN/int8/quant_dtype_cast_int8.c:180-203 (non-ARM branch): float reciprocal, float multiply, float add of the
 * converted zero point, round half away via double round(), conversion to int, clamp.  A NaN or a value beyond the
 * int range converts to INT_MIN on x86 (cvttsd2si) and so clamps to -128. */
void orc_quantize_fp32_int8(const float *x, int8_t *q, float scale, int32_t zp, int64_t n) {
  volatile float inv = 1.0f / scale;
  const float zpf = (float)zp;
  for (int64_t i = 0; i < n; ++i) {
    float v = x[i];
    int32_t t;
    if (v == INFINITY) {
      t = 127;
    } else if (v == -INFINITY) {
      t = -128;
    } else {
      volatile float prod = v * inv;
      volatile float sum = prod + zpf;
      double r = round((double)sum);
      if (!(r >= -2147483648.0 && r <= 2147483647.0)) {
        t = INT32_MIN; /* out-of-range or NaN double -> int conversion on x86-64 */
      } else {
        t = (int32_t)r;
      }
      if (t > 127) t = 127;
      if (t < -128) t = -128;
    }
    q[i] = (int8_t)t;
  }
}

/* LK/int8/dynamic_quant.cc:288-366 for the per-tensor case (axis_num_ == 0) */
int orc_dynamic_quant(const float *x, int64_t n, int symmetric, int8_t *q, double *scale, int32_t *zp) {
  float mn = FLT_MAX, mx = -FLT_MAX;
  orc_minmax_fp32(x, n, &mn, &mx);
  orc_dynquant_params(mn, mx, symmetric, scale, zp);
  orc_quantize_fp32_int8(x, q, (float)*scale, *zp, n);
  return 0;
}

/* Dynamic-quant MatMul: NN/int8/dynamic_matmul_int8.c:99-143 driven by LK/int8/matmul_dynamic_int8.cc:40-65.
 * value = sum(a*b) - zw*sum(a) - zx*sum(b) + K*zx*zw in wrapping int32 over the true K; the per-channel case still
 * uses the single zero point zw[0] (matmul_dynamic_int8.cc:52).  dst = (sx*sw) * (float)value, then + bias, then
 * the activation -- three separately rounded float operations. */
/* DynamicQuantCPUKernel with prefer_axes (LK/int8/dynamic_quant.cc:59-94 ReSize, :118-143 CalculateMinMax, :188-218
 * CalculatePerChannelScaleZp, :236-246 QuantData): after the preferred axes lead, the tensor is `segments` contiguous
 * runs of `unit` elements, each with its own min/max, scale and zero point.  The scale / zero-point formulas are
 * those of the per-tensor case. */
int orc_dynamic_quant_segments(const float *x, int64_t segments, int64_t unit, int symmetric, int8_t *q,
                               double *scales, int32_t *zps) {
  if (segments < 1 || unit < 1) return -1;
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int64_t s = 0; s < segments; ++s) {
    float mn = FLT_MAX, mx = -FLT_MAX;
    orc_minmax_fp32(x + s * unit, unit, &mn, &mx);
    orc_dynquant_params(mn, mx, symmetric, &scales[s], &zps[s]);
    orc_quantize_fp32_int8(x + s * unit, q + s * unit, (float)scales[s], zps[s], unit);
  }
  return 0;
}

static int dyn_mm(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k, int b_transpose,
                  float fsx, const float *sx_rows, int zx, const double *sw, const int32_t *zw, int nfilt,
                  int act_type);

int orc_dynamic_matmul(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                       int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt,
                       int act_type) {
  return dyn_mm(a, w, bias, c, m, n, k, b_transpose, (float)sx, NULL, zx, sw, zw, nfilt, act_type);
}

/* input_per_channel_: one input scale per row, a single input zero point -- the first one
 * (LK/int8/matmul_dynamic_int8.cc:61-62, NN/int8/dynamic_matmul_int8.c:126-128) */
int orc_dynamic_matmul_rows(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                            int b_transpose, const float *sx_rows, int zx, const double *sw, const int32_t *zw,
                            int nfilt, int act_type) {
  if (sx_rows == NULL) return -1;
  return dyn_mm(a, w, bias, c, m, n, k, b_transpose, 0.0f, sx_rows, zx, sw, zw, nfilt, act_type);
}

static int dyn_mm(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k, int b_transpose,
                  float fsx, const float *sx_rows, int zx, const double *sw, const int32_t *zw, int nfilt,
                  int act_type) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != n)) return -1;
  const int peroc = nfilt > 1;
  const int32_t z = zw[0];
  int8_t *wt = NULL;
  const int8_t *wnk = w;
  if (!b_transpose) {
    wt = (int8_t *)malloc((size_t)n * (size_t)k + 1);
    if (!wt) return -1;
    for (int kk = 0; kk < k; ++kk)
      for (int cc = 0; cc < n; ++cc) wt[(size_t)cc * k + kk] = w[(size_t)kk * n + cc];
    wnk = wt;
  }
  int32_t *wsum = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
  if (!wsum) return -1;
  for (int cc = 0; cc < n; ++cc) {
    int32_t s = 0;
    for (int kk = 0; kk < k; ++kk) s += wnk[(size_t)cc * k + kk];
    wsum[cc] = s;
  }
#pragma omp parallel for num_threads(g_threads) schedule(static)
  for (int r = 0; r < m; ++r) {
    const int8_t *ar = a + (size_t)r * k;
    int32_t asum = 0;
    for (int kk = 0; kk < k; ++kk) asum += ar[kk];
    for (int cc = 0; cc < n; ++cc) {
      const int8_t *wr = wnk + (size_t)cc * k;
      int32_t s0 = 0;
      for (int kk = 0; kk < k; ++kk) s0 += (int32_t)ar[kk] * (int32_t)wr[kk];
      int32_t s1 = wmul(z, asum), s2 = wmul(zx, wsum[cc]), s3 = wmul(wmul(k, zx), z);
      int32_t value = wadd(wsub(wsub(s0, s1), s2), s3);
      volatile float ms = (sx_rows ? sx_rows[r] : fsx) * (float)sw[peroc ? cc : 0];
      volatile float d = ms * (float)value;
      if (bias) d = d + bias[cc];
      float o = d;
      if (act_type == ORC_ACT_RELU) {
        o = (0 > o) ? 0 : o; /* MSMAX(0, x): 0 > x ? 0 : x -- a NaN survives */
      } else if (act_type == ORC_ACT_RELU6) {
        o = (0 > o) ? 0 : o;
        o = (6 < o) ? 6 : o;
      }
      c[(size_t)r * n + cc] = o;
    }
  }
  free(wsum);
  free(wt);
  return 0;
}
