/*
 * TEST INFRASTRUCTURE ONLY.  Driver over the REAL nnacl int8 kernels, compiled from the reference tree where it
 * lies (see oracle/Makefile) into oracle/_ref/libnnacl_ref.so.  It performs, in plain C with pthreads, the same
 * call sequence each Lite CPU wrapper performs on x86 (non-ARM branches) so the results and the timing are those
 * of the reference's CPU path.  The wrappers themselves are C++ inside litert and cannot be compiled here; the
 * few scalar lines they contribute (multiplier derivation, dynamic-quant scale/zero point) are written out below
 * with a citation each.
 *
 *   LK/ = mindspore/lite/src/litert/kernel/cpu/      NN/ = mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/
 */
#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "nnacl/base/conv1x1_base.h"
#include "nnacl/conv_parameter.h"
#include "nnacl/int8/conv1x1_int8.h"
#include "nnacl/int8/conv_depthwise_int8.h"
#include "nnacl/int8/conv_int8.h"
#include "nnacl/int8/dynamic_matmul_int8.h"
#include "nnacl/int8/dynamic_quant_int8.h"
#include "nnacl/int8/fixed_point.h"
#include "nnacl/int8/matmul_int8.h"
#include "nnacl/int8/pack_int8.h"
#include "nnacl/int8/quant_dtype_cast_int8.h"
#include "nnacl/int8/quantize.h"
#include "nnacl/matmul_parameter.h"

typedef struct ref_conv_shape {
  int batch, in_h, in_w, in_c;
  int out_h, out_w, out_c;
  int kernel_h, kernel_w, stride_h, stride_w, dilation_h, dilation_w;
  int pad_u, pad_l;
} ref_conv_shape;

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

/* ---- tiny stand-in for ParallelLaunch (mindspore/core/mindrt/src/thread/threadpool.cc:298): run f(ctx, task)
 *      for task in [0, tasks) on `tasks` threads and join ---- */
typedef void (*task_fn)(void *ctx, int task);
typedef struct launch_arg {
  task_fn fn;
  void *ctx;
  int task;
} launch_arg;
static void *launch_tramp(void *p) {
  launch_arg *a = (launch_arg *)p;
  a->fn(a->ctx, a->task);
  return NULL;
}
static void parallel_launch(task_fn fn, void *ctx, int tasks) {
  if (tasks <= 1) {
    fn(ctx, 0);
    return;
  }
  pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)tasks);
  launch_arg *args = (launch_arg *)malloc(sizeof(launch_arg) * (size_t)tasks);
  for (int i = 0; i < tasks; ++i) {
    args[i].fn = fn;
    args[i].ctx = ctx;
    args[i].task = i;
    pthread_create(&th[i], NULL, launch_tramp, &args[i]);
  }
  for (int i = 0; i < tasks; ++i) pthread_join(th[i], NULL);
  free(th);
  free(args);
}

/* LK/int8/matmul_base_int8.cc:258-266 and LK/base/convolution_base.cc:416-427 */
static void derive_multipliers(double sx, const double *sw, int nfilt, double so, int32_t *mult, int32_t *ls,
                               int32_t *rs) {
  QuantArg in, out;
  in.scale_ = sx;
  out.scale_ = so;
  for (int i = 0; i < nfilt; ++i) {
    float fs = sw[i];
    const double in_scale = (double)(in.scale_ * fs);
    double real = in_scale / (double)(out.scale_);
    QuantizeRoundParameterWithDoublePrecision(real, &mult[i], &ls[i], &rs[i]);
  }
}

/* ------------------------------------------------------------------------------------------------------------
 * Full-quant MatMul / FullConnection: LK/int8/matmul_base_int8.cc:129-150 (RunImpl), :275-336, :360-415, :530-571
 * ------------------------------------------------------------------------------------------------------------ */
typedef struct mm_ctx {
  const int8_t *pack_a, *pack_b;
  int8_t *c;
  int row, col, deep16, stride_cols;
  const int32_t *asum, *wsum;
  int32_t amin, amax, zo;
  const int32_t *mult, *ls, *rs, *zw;
  int peroc;
} mm_ctx;

static void mm_task(void *p, int task) {
  mm_ctx *x = (mm_ctx *)p;
  int cur_stride = task * x->stride_cols;
  int cur_oc = x->col - cur_stride;
  if (cur_oc > x->stride_cols) cur_oc = x->stride_cols;
  if (cur_oc <= 0) return;
  const int32_t *cl = x->peroc ? x->ls + cur_stride : x->ls;
  const int32_t *cr = x->peroc ? x->rs + cur_stride : x->rs;
  const int32_t *cm = x->peroc ? x->mult + cur_stride : x->mult;
  const int32_t *cz = x->peroc ? x->zw + cur_stride : x->zw;
  MatmulInt8Opt(x->pack_a, x->pack_b + (size_t)cur_stride * x->deep16, x->c + cur_stride, x->row, cur_oc, x->deep16,
                x->asum, x->wsum + cur_stride, x->amin, x->amax, x->zo, cm, cl, cr, (size_t)x->col, (size_t)x->peroc,
                cz);
}

int ref_matmul_int8(const int8_t *a, const int8_t *w, const int32_t *bias, int8_t *c, int m, int n, int k,
                    int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so,
                    int zo, int act_type, int threads, double *run_seconds) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != n)) return -1;
  const int peroc = nfilt > 1;
  const int row4 = UP_ROUND(m, C4NUM), col4 = UP_ROUND(n, C4NUM), deep16 = UP_ROUND(k, C16NUM);
  int32_t *mult = calloc((size_t)nfilt, 4), *ls = calloc((size_t)nfilt, 4), *rs = calloc((size_t)nfilt, 4);
  int32_t amin, amax;
  /* Prepare: InitQuantParam */
  derive_multipliers(sx, sw, nfilt, so, mult, ls, rs);
  CalculateActivationRangeQuantized(act_type == ActType_Relu, act_type == ActType_Relu6, zo, (float)so, &amin, &amax);
  /* ReSize: InitTmpBuffer + TransferB */
  int8_t *pack_a = calloc((size_t)row4 * deep16 + 1, 1);
  int8_t *pack_b = calloc((size_t)col4 * deep16 + 1, 1);
  int32_t *asum = calloc((size_t)row4 + 1, 4);
  int32_t *wsum = calloc((size_t)col4 + 1, 4);
  if (b_transpose) {
    RowMajor2Row16x4MajorInt8(w, pack_b, n, k);
    CalcWeightBiasSums(w, k, n, zx, zw, bias, wsum, ColMajor, peroc);
  } else {
    RowMajor2Col16x4MajorInt8(w, pack_b, k, n);
    CalcWeightBiasSums(w, k, n, zx, zw, bias, wsum, RowMajor, peroc);
  }
  int thread_count = threads < UP_DIV(col4, C4NUM) ? threads : UP_DIV(col4, C4NUM);
  if (thread_count < 1) thread_count = 1;
  int thread_stride = UP_DIV(UP_DIV(col4, C4NUM), thread_count);
  /* Run */
  double t0 = now_s();
  RowMajor2Row16x4MajorInt8(a, pack_a, m, k);
  CalcInputSums(a, m, k, peroc ? 1 : zw[0], asum, RowMajor);
  mm_ctx x = {pack_a, pack_b, c, m, n, deep16, thread_stride * C4NUM, asum, wsum, amin, amax, zo, mult, ls, rs, zw,
              peroc};
  parallel_launch(mm_task, &x, thread_count);
  if (run_seconds) *run_seconds = now_s() - t0;
  free(mult);
  free(ls);
  free(rs);
  free(pack_a);
  free(pack_b);
  free(asum);
  free(wsum);
  return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * Conv2D int8, group 1.  Selection as LK/int8/convolution_int8_creator.cc:76-99 minus the Winograd branch
 * (3x3 s1 d1 is rejected here: the reference runs an inexact integer Winograd there on x86).
 * ------------------------------------------------------------------------------------------------------------ */
typedef struct conv_quant_store {
  QuantArg in_q, out_q;
  QuantArg *filt_q;
  int32_t *mult, *ls, *rs;
  int32_t amin, amax;
  double *real;
} conv_quant_store;

/* LK/base/convolution_base.cc:246-292 (SetIfPerChannel), :330-377, :379-430, :460-499 */
static void fill_conv_param(ConvParameter *cp, conv_quant_store *qs, const ref_conv_shape *s, double sx, int zx,
                            const double *sw, const int32_t *zw, int nfilt, double so, int zo, int act_type,
                            int threads) {
  memset(cp, 0, sizeof(*cp));
  cp->kernel_h_ = s->kernel_h;
  cp->kernel_w_ = s->kernel_w;
  cp->stride_h_ = s->stride_h;
  cp->stride_w_ = s->stride_w;
  cp->dilation_h_ = s->dilation_h;
  cp->dilation_w_ = s->dilation_w;
  cp->pad_u_ = s->pad_u;
  cp->pad_l_ = s->pad_l;
  cp->group_ = 1;
  cp->input_batch_ = s->batch;
  cp->input_h_ = s->in_h;
  cp->input_w_ = s->in_w;
  cp->input_channel_ = s->in_c;
  cp->output_batch_ = s->batch;
  cp->output_h_ = s->out_h;
  cp->output_w_ = s->out_w;
  cp->output_channel_ = s->out_c;
  cp->thread_num_ = threads;
  cp->act_type_ = (ActType)act_type;
  qs->in_q.scale_ = sx;
  qs->in_q.zp_ = zx;
  qs->out_q.scale_ = so;
  qs->out_q.zp_ = zo;
  qs->filt_q = calloc((size_t)nfilt, sizeof(QuantArg));
  for (int i = 0; i < nfilt; ++i) {
    qs->filt_q[i].scale_ = sw[i];
    qs->filt_q[i].zp_ = zw[i];
  }
  qs->mult = calloc((size_t)nfilt, 4);
  qs->ls = calloc((size_t)nfilt, 4);
  qs->rs = calloc((size_t)nfilt, 4);
  qs->real = calloc((size_t)nfilt, 8);
  derive_multipliers(sx, sw, nfilt, so, qs->mult, qs->ls, qs->rs);
  CalculateActivationRangeQuantized(act_type == ActType_Relu, act_type == ActType_Relu6, zo, qs->out_q.scale_,
                                    &qs->amin, &qs->amax);
  ConvQuantArg *q = &cp->conv_quant_arg_;
  q->round_mode_ = Rounding_Away_from_zero;
  q->quant_multiplier_mode_ = Method_DoublePrecision;
  q->input_quant_args_ = &qs->in_q;
  q->filter_quant_args_ = qs->filt_q;
  q->output_quant_args_ = &qs->out_q;
  q->real_multiplier_ = qs->real;
  q->left_shift_ = qs->ls;
  q->right_shift_ = qs->rs;
  q->quant_multiplier_ = qs->mult;
  q->out_act_min_ = &qs->amin;
  q->out_act_max_ = &qs->amax;
  q->input_arg_num_ = 1;
  q->filter_arg_num_ = (size_t)nfilt;
  q->output_arg_num_ = 1;
  q->per_channel_ = nfilt != 1 ? FILTER_PER_CHANNEL : 0;
}

static void free_conv_quant(conv_quant_store *qs) {
  free(qs->filt_q);
  free(qs->mult);
  free(qs->ls);
  free(qs->rs);
  free(qs->real);
}

/* ---- im2col path: LK/int8/convolution_int8.cc:30-51 (x86: tile 8, support_optimize_ stays true), :53-180, :229-263 */
typedef struct im2col_ctx {
  int8_t *in, *packed_in, *matmul_in, *packed_w, *out;
  int32_t *bias2, *zw_arr, *isum;
  ConvParameter *cp;
} im2col_ctx;
static void im2col_task(void *p, int task) {
  im2col_ctx *x = (im2col_ctx *)p;
  ConvInt8(x->in, x->packed_in, x->matmul_in, x->packed_w, x->bias2, x->out, x->zw_arr, x->isum, task, x->cp, NULL,
           true);
}

static int ref_conv_im2col(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out,
                           const ref_conv_shape *s, ConvParameter *cp, int zx, const int32_t *zw, int nfilt,
                           int threads, double *run_seconds) {
  const int peroc = nfilt != 1;
  const int oc = s->out_c, kplane = s->kernel_h * s->kernel_w, kdim = kplane * s->in_c;
  const int up_oc = UP_ROUND(oc, C8NUM), up_deep = UP_ROUND(kdim, C4NUM);
  const int tile = 8;
  cp->tile_num_ = tile;
  int8_t *packed_w = calloc((size_t)up_oc * up_deep + 1, 1);
  RowMajor2Row8x4MajorInt8(w, packed_w, oc, kdim);
  int32_t *bias2 = calloc((size_t)up_oc, 4);
  if (bias) memcpy(bias2, bias, (size_t)oc * 4);
  int32_t *zw_arr = peroc ? calloc((size_t)oc, 4) : NULL;
  for (int o = 0; o < oc; ++o) { /* convolution_int8.cc:121-142 */
    int32_t filter_zp = zw[0];
    if (peroc) {
      filter_zp = zw[o];
      zw_arr[o] = filter_zp;
    }
    int32_t weight_sum_value = up_deep * filter_zp;
    for (int i = 0; i < kdim; i++) weight_sum_value += w[(size_t)o * kdim + i] - filter_zp;
    bias2[o] += filter_zp * zx * up_deep - weight_sum_value * zx;
  }
  size_t isum_n = peroc ? (size_t)up_oc * tile * threads : (size_t)tile * threads;
  int32_t *isum = calloc(isum_n + 1, 4);
  double t0 = now_s();
  int8_t *matmul_in = malloc((size_t)threads * tile * kdim + 1); /* InitTmpBuffer, per Run */
  int8_t *packed_in = malloc((size_t)up_deep * threads * tile + 1);
  im2col_ctx x = {(int8_t *)in, packed_in, matmul_in, packed_w, out, bias2, zw_arr, isum, cp};
  parallel_launch(im2col_task, &x, threads);
  free(matmul_in);
  free(packed_in);
  if (run_seconds) *run_seconds = now_s() - t0;
  free(packed_w);
  free(bias2);
  free(zw_arr);
  free(isum);
  return 0;
}

/* ---- 1x1 path: LK/int8/convolution_1x1_int8.cc:139-141 (x86: support_optimize_ false), :158-267, :359-397,
 *      :446-472 (RunArmHw), :524-550 (RunArmOc), :572-621 (Run) */
typedef struct c11_ctx {
  int8_t *input_ptr, *output_ptr, *packed_in, *packed_w;
  int32_t *isum, *bias2, *ls, *rs, *mult, *zw_arr;
  ConvParameter *cp;
  int row, col, deep, deep16, peroc;
  int thread_stride_hw, thread_stride_oc;
} c11_ctx;

static void c11_hw_task(void *p, int task) {
  c11_ctx *x = (c11_ctx *)p;
  int cur_stride = x->thread_stride_hw * C4NUM;
  int res_stride = x->row - task * x->thread_stride_hw * C4NUM;
  int cur_hw = cur_stride < res_stride ? cur_stride : res_stride;
  if (cur_hw <= 0) return;
  int8_t *hw_in = x->input_ptr + (size_t)task * x->thread_stride_hw * C4NUM * x->deep;
  int8_t *hw_out = x->output_ptr + (size_t)task * x->thread_stride_hw * C4NUM * x->col;
  int8_t *hw_packed = x->packed_in + (size_t)task * x->thread_stride_hw * C4NUM * x->deep16;
  int32_t *hw_sum = x->isum + (size_t)task * x->thread_stride_hw * C4NUM;
  RowMajor2Row16x4MajorInt8(hw_in, hw_packed, cur_hw, x->deep);
  PackInputSum16x4PerLayer(hw_packed, hw_sum, x->peroc ? 1 : x->cp->conv_quant_arg_.filter_quant_args_[0].zp_,
                           UP_ROUND(cur_hw, C4NUM), x->deep16);
  Conv1x1Int8(hw_packed, x->packed_w, hw_out, hw_sum, x->bias2, cur_hw, x->col, x->deep16, x->ls, x->rs, x->mult,
              x->cp, x->zw_arr);
}

static void c11_oc_task(void *p, int task) {
  c11_ctx *x = (c11_ctx *)p;
  int stride = x->thread_stride_oc * C4NUM;
  int cur_stride = task * stride;
  int res_stride = x->col - cur_stride;
  int cur_oc = stride < res_stride ? stride : res_stride;
  if (cur_oc <= 0) return;
  int32_t *cl = x->peroc ? x->ls + cur_stride : x->ls;
  int32_t *cr = x->peroc ? x->rs + cur_stride : x->rs;
  int32_t *cm = x->peroc ? x->mult + cur_stride : x->mult;
  int32_t *cz = x->peroc ? x->zw_arr + cur_stride : x->zw_arr;
  Conv1x1Int8(x->packed_in, x->packed_w + (size_t)cur_stride * x->deep16, x->output_ptr + cur_stride, x->isum,
              x->bias2 + cur_stride, x->row, cur_oc, x->deep16, cl, cr, cm, x->cp, cz);
}

static int ref_conv_1x1(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const ref_conv_shape *s,
                        ConvParameter *cp, conv_quant_store *qs, int zx, const int32_t *zw, int nfilt, int threads,
                        double *run_seconds) {
  const int peroc = nfilt != 1;
  const int ic = s->in_c, oc = s->out_c;
  const int row = s->out_h * s->out_w, deep16 = UP_ROUND(ic, C16NUM), round_oc = UP_ROUND(oc, C4NUM);
  int8_t *packed_w = calloc((size_t)deep16 * round_oc + 1, 1);
  RowMajor2Row16x4MajorInt8(w, packed_w, oc, ic);
  int32_t *bias2 = calloc((size_t)round_oc, 4);
  if (bias) memcpy(bias2, bias, (size_t)oc * 4);
  for (int o = 0; o < oc; ++o) { /* InitBiasByzp :158-176 */
    int32_t weight_sum_value = 0;
    int32_t filter_zp = peroc ? zw[o] : zw[0];
    for (int i = 0; i < ic; i++) weight_sum_value += w[(size_t)o * ic + i];
    bias2[o] += filter_zp * zx * ic - weight_sum_value * zx;
  }
  int32_t *zw_arr = NULL, *ls = qs->ls, *rs = qs->rs, *mult = qs->mult;
  if (peroc) { /* :178-215: arrays padded to round_oc */
    zw_arr = calloc((size_t)round_oc, 4);
    ls = calloc((size_t)round_oc, 4);
    rs = calloc((size_t)round_oc, 4);
    mult = calloc((size_t)round_oc, 4);
    memcpy(zw_arr, zw, (size_t)oc * 4);
    memcpy(ls, qs->ls, (size_t)oc * 4);
    memcpy(rs, qs->rs, (size_t)oc * 4);
    memcpy(mult, qs->mult, (size_t)oc * 4);
  }
  /* InitParam :359-413 */
  const int pre_trans = (s->pad_u != 0 || s->pad_l != 0 || s->stride_h != 1 || s->stride_w != 1);
  int8_t *gather = NULL;
  if (pre_trans) gather = calloc((size_t)row * ic + 1, 1); /* memset 0 once */
  int hw_thread_count = UP_DIV(row, C4NUM), oc_thread_count = UP_DIV(oc, C4NUM);
  int thread_count_hw = threads < hw_thread_count ? threads : hw_thread_count;
  int thread_count_oc = threads < oc_thread_count ? threads : oc_thread_count;
  if (thread_count_hw < 1) thread_count_hw = 1;
  if (thread_count_oc < 1) thread_count_oc = 1;
  int parallel_by_oc = oc_thread_count > threads;
  c11_ctx x;
  memset(&x, 0, sizeof(x));
  x.packed_w = packed_w;
  x.bias2 = bias2;
  x.ls = ls;
  x.rs = rs;
  x.mult = mult;
  x.zw_arr = zw_arr;
  x.cp = cp;
  x.row = row;
  x.col = oc;
  x.deep = ic;
  x.deep16 = deep16;
  x.peroc = peroc;
  x.thread_stride_hw = UP_DIV(hw_thread_count, thread_count_hw);
  x.thread_stride_oc = UP_DIV(oc_thread_count, thread_count_oc);
  double t0 = now_s();
  x.isum = malloc(((size_t)UP_ROUND(row, C4NUM) + 1) * 4); /* InitRunBuf, per Run */
  x.packed_in = malloc((size_t)UP_ROUND(row, C4NUM) * deep16 + 1);
  for (int b = 0; b < s->batch; ++b) {
    const int8_t *src = in + (size_t)b * s->in_h * s->in_w * ic;
    x.output_ptr = out + (size_t)b * row * oc;
    if (pre_trans) {
      Conv1x1InputPack(src, gather, cp, sizeof(int8_t));
      x.input_ptr = gather;
    } else {
      x.input_ptr = (int8_t *)src;
    }
    if (parallel_by_oc) {
      RowMajor2Row16x4MajorInt8(x.input_ptr, x.packed_in, row, ic);
      PackInputSum16x4PerLayer(x.packed_in, x.isum, peroc ? 1 : zw[0], UP_ROUND(row, C4NUM), deep16);
      parallel_launch(c11_oc_task, &x, thread_count_oc);
    } else {
      parallel_launch(c11_hw_task, &x, thread_count_hw);
    }
  }
  free(x.isum);
  free(x.packed_in);
  if (run_seconds) *run_seconds = now_s() - t0;
  if (peroc) {
    free(zw_arr);
    free(ls);
    free(rs);
    free(mult);
  }
  free(gather);
  free(packed_w);
  free(bias2);
  return 0;
}

static int conv_int8_impl(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const ref_conv_shape *s,
                          double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo,
                          int act_type, int threads, double *run_seconds, int winograd_guard) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != s->out_c)) return -1;
  if (winograd_guard && s->kernel_h == 3 && s->kernel_w == 3 && s->stride_h == 1 && s->stride_w == 1 &&
      s->dilation_h == 1 && s->dilation_w == 1)
    return -2; /* Winograd branch of the reference: not an exact integer convolution */
  if (threads < 1) threads = 1;
  ConvParameter cp;
  conv_quant_store qs;
  fill_conv_param(&cp, &qs, s, sx, zx, sw, zw, nfilt, so, zo, act_type, threads);
  int rc;
  if (s->kernel_h == 1 && s->kernel_w == 1) {
    rc = ref_conv_1x1(in, w, bias, out, s, &cp, &qs, zx, zw, nfilt, threads, run_seconds);
  } else {
    rc = ref_conv_im2col(in, w, bias, out, s, &cp, zx, zw, nfilt, threads, run_seconds);
  }
  free_conv_quant(&qs);
  return rc;
}

/* Kernel selection as on x86 (mindspore/lite/src/litert/kernel/cpu/int8/convolution_int8_creator.cc:81-94): dense
 * 3x3 stride-1 dilation-1 goes to the Winograd kernel there and is refused here. */
int ref_conv_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const ref_conv_shape *s,
                  double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo, int act_type,
                  int threads, double *run_seconds) {
  return conv_int8_impl(in, w, bias, out, s, sx, zx, sw, zw, nfilt, so, zo, act_type, threads, run_seconds, 1);
}

/* Kernel selection as on ARM64 cores with the dot-product extension (same lines: ConvolutionInt8CPUKernel for every
 * dense kernel size): ConvInt8 also for 3x3 stride 1.  The C code of ConvInt8 is the same on every platform. */
int ref_conv_int8_as_arm64_sdot(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out,
                                const ref_conv_shape *s, double sx, int zx, const double *sw, const int32_t *zw,
                                int nfilt, double so, int zo, int act_type, int threads, double *run_seconds) {
  return conv_int8_impl(in, w, bias, out, s, sx, zx, sw, zw, nfilt, so, zo, act_type, threads, run_seconds, 0);
}

/* ------------------------------------------------------------------------------------------------------------
 * Depthwise: LK/int8/convolution_depthwise_int8.cc:33-105,129,142-197
 * ------------------------------------------------------------------------------------------------------------ */
typedef struct dw_ctx {
  int8_t *out;
  int32_t *row_buffer;
  const int8_t *in;
  const int16_t *w16;
  const int32_t *bias;
  ConvParameter *cp;
} dw_ctx;
static void dw_task(void *p, int task) {
  dw_ctx *x = (dw_ctx *)p;
  ConvDwInt8(x->out, x->row_buffer + (size_t)x->cp->output_w_ * x->cp->output_channel_ * task, x->in, x->w16, x->bias,
             x->cp, task);
}

int ref_conv_dw_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const ref_conv_shape *s,
                     double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo,
                     int act_type, int threads, double *run_seconds) {
  const int ch = s->out_c, plane = s->kernel_h * s->kernel_w;
  if (s->in_c != ch || nfilt < 1 || (nfilt > 1 && nfilt != ch)) return -1;
  if (threads < 1) threads = 1;
  ConvParameter cp;
  conv_quant_store qs;
  fill_conv_param(&cp, &qs, s, sx, zx, sw, zw, nfilt, so, zo, act_type, threads);
  cp.group_ = ch;
  cp.thread_num_ = threads < s->out_h ? threads : s->out_h;
  int8_t *tmp = malloc((size_t)ch * plane + 1);
  PackNCHWToNHWCInt8(w, tmp, 1, plane, ch);
  int16_t *w16 = malloc(((size_t)ch * plane + 1) * 2);
  if (nfilt != 1) {
    for (int i = 0; i < plane; i++)
      for (int c = 0; c < ch; c++) w16[i * ch + c] = (int16_t)(tmp[i * ch + c] - zw[c]);
  } else {
    for (int i = 0; i < plane * ch; i++) w16[i] = (int16_t)(tmp[i] - zw[0]);
  }
  free(tmp);
  int32_t *b2 = calloc((size_t)ch, 4);
  if (bias) memcpy(b2, bias, (size_t)ch * 4);
  double t0 = now_s();
  int32_t *row_buffer = malloc(((size_t)cp.thread_num_ * s->out_w * ch + 1) * 4);
  dw_ctx x = {out, row_buffer, in, w16, b2, &cp};
  parallel_launch(dw_task, &x, cp.thread_num_);
  free(row_buffer);
  if (run_seconds) *run_seconds = now_s() - t0;
  free(w16);
  free(b2);
  free_conv_quant(&qs);
  return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * DynamicQuant per tensor: LK/int8/dynamic_quant.cc:59-66,96-116 (buckets), :118-143, :156-186, :220-234, :288-366
 * ------------------------------------------------------------------------------------------------------------ */
typedef struct dq_ctx {
  const float *x;
  int8_t *q;
  int ele_num, unit_num, unit_segment_num;
  float *real_min, *real_max;
  float scale;
  int32_t zp;
} dq_ctx;

static void dq_minmax_task(void *p, int task) {
  dq_ctx *d = (dq_ctx *)p;
  int task_unit = d->unit_segment_num * d->unit_num;
  int offset = task * task_unit;
  int remain = d->ele_num - offset;
  if (task_unit <= remain) {
    for (int i = 0; i < d->unit_segment_num; ++i)
      CalculateMinMaxFp32(d->x + offset + i * d->unit_num, d->unit_num, &d->real_min[task * d->unit_segment_num + i],
                          &d->real_max[task * d->unit_segment_num + i]);
  } else {
    int segment_num = remain / d->unit_num;
    int remain_ele_num = remain - segment_num * d->unit_num;
    for (int i = 0; i < segment_num; ++i)
      CalculateMinMaxFp32(d->x + offset + i * d->unit_num, d->unit_num, &d->real_min[task * d->unit_segment_num + i],
                          &d->real_max[task * d->unit_segment_num + i]);
    if (remain_ele_num == 0) return;
    CalculateMinMaxFp32(d->x + offset + segment_num * d->unit_num, remain_ele_num,
                        &d->real_min[task * d->unit_segment_num + segment_num],
                        &d->real_max[task * d->unit_segment_num + segment_num]);
  }
}

static void dq_quant_task(void *p, int task) {
  dq_ctx *d = (dq_ctx *)p;
  int task_unit = d->unit_segment_num * d->unit_num;
  int offset = task * task_unit;
  int remain = d->ele_num - offset;
  if (task_unit > remain) task_unit = remain;
  DoQuantizeFp32ToInt8(d->x + offset, d->q + offset, d->scale, d->zp, task_unit, (int32_t)INT8_MIN, (int32_t)INT8_MAX);
}

int ref_dynamic_quant(const float *x, int n, int symmetric, int8_t *q, double *scale_out, int32_t *zp_out, int threads,
                      double *run_seconds) {
  if (threads < 1) threads = 1;
  int segment_num = n / 512 < 8 ? n / 512 : 8; /* kBucketNums, kMinNums */
  if (segment_num <= 0) segment_num = 1;
  dq_ctx d;
  d.x = x;
  d.q = q;
  d.ele_num = n;
  d.real_min = malloc(sizeof(float) * (size_t)segment_num);
  d.real_max = malloc(sizeof(float) * (size_t)segment_num);
  int thread_num = segment_num < threads ? segment_num : threads;
  d.unit_num = UP_DIV(n, segment_num);
  d.unit_segment_num = UP_DIV(segment_num, thread_num);
  double t0 = now_s();
  for (int i = 0; i < segment_num; ++i) {
    d.real_min[i] = FLT_MAX;
    d.real_max[i] = -FLT_MAX;
  }
  parallel_launch(dq_minmax_task, &d, thread_num);
  /* CalculatePerlayerScaleZp :156-186 */
  float real_min = FLT_MAX, real_max = -FLT_MAX;
  for (int i = 0; i < segment_num; ++i) {
    real_min = (d.real_min[i] < real_min) ? d.real_min[i] : real_min;
    real_max = (d.real_max[i] > real_max) ? d.real_max[i] : real_max;
  }
  double scale;
  int zp = 0;
  if (!symmetric) {
    float range = real_max - real_min;
    if (range <= 0) range = 0.01f;
    scale = range / 255;
    zp = (int)round(INT8_MIN - real_min / scale);
  } else {
    float amax = fabsf(real_max), amin = fabsf(real_min);
    float mx = amax < amin ? amin : amax;
    scale = 2 * mx / 254;
  }
  d.scale = (float)scale; /* DoQuantizeFp32ToInt8 takes a float scale */
  d.zp = zp;
  parallel_launch(dq_quant_task, &d, thread_num);
  if (run_seconds) *run_seconds = now_s() - t0;
  *scale_out = scale;
  *zp_out = zp;
  free(d.real_min);
  free(d.real_max);
  return 0;
}

/* ------------------------------------------------------------------------------------------------------------
 * Dynamic-quant MatMul: LK/int8/matmul_dynamic_int8.cc:40-65,86-147; base LK/int8/matmul_dynamic_base_int8.cc
 * ------------------------------------------------------------------------------------------------------------ */
/* DynamicQuantCPUKernel with prefer_axes: CalculateMinMaxFp32 and DoQuantizeFp32ToInt8 per segment, scale and zero
 * point per segment as CalculatePerChannelScaleZp derives them (LK/int8/dynamic_quant.cc:188-218).  Single thread per
 * segment, as in the wrapper. */
int ref_dynamic_quant_segments(const float *x, int segments, int unit, int symmetric, int8_t *q, double *scales,
                               int32_t *zps, int threads, double *run_seconds) {
  (void)threads;
  if (segments < 1 || unit < 1) return -1;
  double t0 = now_s();
  for (int s = 0; s < segments; ++s) {
    float real_min = FLT_MAX, real_max = -FLT_MAX;
    CalculateMinMaxFp32(x + (size_t)s * unit, unit, &real_min, &real_max);
    double scale;
    int zp = 0;
    if (!symmetric) {
      float range = real_max - real_min;
      if (range <= 0) range = 0.01f;
      scale = range / 255;
      zp = (int)round(INT8_MIN - real_min / scale);
    } else {
      float amax = fabsf(real_max), amin = fabsf(real_min);
      float mx = amax < amin ? amin : amax;
      scale = 2 * mx / 254;
    }
    scales[s] = scale;
    zps[s] = zp;
    DoQuantizeFp32ToInt8(x + (size_t)s * unit, q + (size_t)s * unit, (float)scale, zp, unit, INT8_MIN, INT8_MAX);
  }
  if (run_seconds) *run_seconds = now_s() - t0;
  return 0;
}

typedef struct dm_ctx {
  const int8_t *pack_a, *pack_b;
  const float *bias;
  float *c;
  int row, col, deep, deep16, stride_cols;
  int zx;
  const float *sx;
  const float *swf;
  int zw0, peroc, act_type;
  int per_row; /* input_per_channel_: sx has one entry per row */
} dm_ctx;

static void dm_task(void *p, int task) {
  dm_ctx *x = (dm_ctx *)p;
  int cur_stride = task * x->stride_cols;
  int cur_oc = x->col - cur_stride;
  if (cur_oc > x->stride_cols) cur_oc = x->stride_cols;
  if (cur_oc <= 0) return;
  const float *b = x->bias ? x->bias + cur_stride : NULL;
  const float *fs = x->peroc ? x->swf + cur_stride : x->swf;
  DynamicMatmul4x16x4AIWI(x->pack_a, x->pack_b + (size_t)cur_stride * x->deep16, b, x->c + cur_stride, x->row, cur_oc,
                          x->deep, x->deep16, (size_t)x->col, x->zx, x->sx, fs, x->zw0, x->per_row != 0, x->peroc,
                          (int64_t)x->act_type);
}

static int ref_dyn_mm(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                      int b_transpose, double sx, const float *sx_rows, int zx, const double *sw, const int32_t *zw,
                      int nfilt, int act_type, int threads, double *run_seconds);

int ref_dynamic_matmul(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                       int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt,
                       int act_type, int threads, double *run_seconds) {
  return ref_dyn_mm(a, w, bias, c, m, n, k, b_transpose, sx, NULL, zx, sw, zw, nfilt, act_type, threads, run_seconds);
}

int ref_dynamic_matmul_rows(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                            int b_transpose, const float *sx_rows, int zx, const double *sw, const int32_t *zw,
                            int nfilt, int act_type, int threads, double *run_seconds) {
  if (sx_rows == NULL) return -1;
  return ref_dyn_mm(a, w, bias, c, m, n, k, b_transpose, 0.0, sx_rows, zx, sw, zw, nfilt, act_type, threads,
                    run_seconds);
}

static int ref_dyn_mm(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                      int b_transpose, double sx, const float *sx_rows, int zx, const double *sw, const int32_t *zw,
                      int nfilt, int act_type, int threads, double *run_seconds) {
  if (nfilt < 1 || (nfilt > 1 && nfilt != n)) return -1;
  if (threads < 1) threads = 1;
  const int peroc = nfilt > 1;
  const int row4 = UP_ROUND(m, C4NUM), col4 = UP_ROUND(n, C4NUM), deep16 = UP_ROUND(k, C16NUM);
  float *swf = malloc(sizeof(float) * (size_t)nfilt);
  for (int i = 0; i < nfilt; ++i) swf[i] = (float)sw[i];
  int8_t *pack_b = calloc((size_t)col4 * deep16 + 1, 1);
  if (b_transpose) {
    RowMajor2Row16x4MajorInt8(w, pack_b, n, k);
  } else {
    RowMajor2Col16x4MajorInt8(w, pack_b, k, n);
  }
  int thread_num = threads < UP_DIV(col4, C4NUM) ? threads : UP_DIV(col4, C4NUM);
  int thread_stride = UP_DIV(UP_DIV(col4, C4NUM), thread_num);
  float sxf = (float)sx;
  double t0 = now_s();
  int8_t *pack_a = malloc((size_t)row4 * deep16 + 1); /* InitMatrixABuffer, per Run */
  memset(pack_a, zx, (size_t)row4 * deep16);
  RowMajor2Row16x4MajorInt8(a, pack_a, m, k);
  dm_ctx x = {pack_a,  pack_b, bias,  c,        m, n, k, deep16, thread_stride * C4NUM, zx, sx_rows ? sx_rows : &sxf,
              swf,     zw[0],  peroc, act_type, sx_rows != NULL};
  parallel_launch(dm_task, &x, thread_num);
  free(pack_a);
  if (run_seconds) *run_seconds = now_s() - t0;
  free(pack_b);
  free(swf);
  return 0;
}

/* ---- shape inference: the real nnacl functions behind Lite's builtin inference ---------------------------------- */
#include "nnacl/infer/conv2d_infer.h"
#include "nnacl/infer/full_connection_infer.h"
#include "nnacl/infer/matmul_infer.h"

static void ref_tensor(TensorC *t, const int *shape, int dims, int dtype) {
  memset(t, 0, sizeof(*t));
  t->data_type_ = dtype;
  t->format_ = Format_NHWC;
  t->shape_size_ = (size_t)dims;
  for (int i = 0; i < dims && i < MAX_SHAPE_SIZE; ++i) t->shape_[i] = shape[i];
}

static int ref_emit_shape(int ret, const TensorC *out, int *out_shape, int *out_dims) {
  *out_dims = (int)out->shape_size_;
  for (size_t i = 0; i < out->shape_size_ && i < MAX_SHAPE_SIZE; ++i) out_shape[i] = out->shape_[i];
  return ret;
}

/* Returns nnacl's own status (NNACL_OK 0, NNACL_INFER_INVALID, or an error). bias_dims 0 = two inputs. */
int ref_infer_matmul(const int *a_shape, int a_dims, const int *b_shape, int b_dims, const int *bias_shape,
                     int bias_dims, int transpose_a, int transpose_b, int *out_shape, int *out_dims) {
  TensorC a, b, bias, out;
  ref_tensor(&a, a_shape, a_dims, kNumberTypeInt8);
  ref_tensor(&b, b_shape, b_dims, kNumberTypeInt8);
  ref_tensor(&bias, bias_shape, bias_dims, kNumberTypeInt32);
  ref_tensor(&out, NULL, 0, kNumberTypeInt8);
  MatMulParameter p;
  memset(&p, 0, sizeof(p));
  p.a_transpose_ = transpose_a != 0;
  p.b_transpose_ = transpose_b != 0;
  const TensorC *in[3] = {&a, &b, &bias};
  TensorC *outs[1] = {&out};
  int ret = MatmulInferShape(in, bias_dims > 0 ? 3 : 2, outs, 1, (OpParameter *)&p);
  return ref_emit_shape(ret, &out, out_shape, out_dims);
}

int ref_infer_fullconnection(const int *a_shape, int a_dims, const int *w_shape, int w_dims, const int *bias_shape,
                             int bias_dims, int has_bias, int use_axis, int axis, int *out_shape, int *out_dims) {
  TensorC a, w, bias, out;
  ref_tensor(&a, a_shape, a_dims, kNumberTypeInt8);
  ref_tensor(&w, w_shape, w_dims, kNumberTypeInt8);
  ref_tensor(&bias, bias_shape, bias_dims, kNumberTypeInt32);
  ref_tensor(&out, NULL, 0, kNumberTypeInt8);
  MatMulParameter p;
  memset(&p, 0, sizeof(p));
  p.has_bias_ = has_bias != 0;
  p.use_axis_ = use_axis != 0;
  p.axis_ = axis;
  const TensorC *in[3] = {&a, &w, &bias};
  TensorC *outs[1] = {&out};
  int ret = FullConnectionInferShape(in, bias_dims > 0 ? 3 : 2, outs, 1, (OpParameter *)&p);
  return ref_emit_shape(ret, &out, out_shape, out_dims);
}

/* cp: kernel_h, kernel_w, stride_h, stride_w, dilation_h, dilation_w, pad_mode, pad_u, pad_d, pad_l, pad_r, group
 * (read, and written back as the reference leaves its ConvParameter). */
int ref_infer_conv2d(const int *in_shape, int in_dims, const int *w_shape, int w_dims, int *cp, int *out_shape,
                     int *out_dims) {
  TensorC in, w, out;
  ref_tensor(&in, in_shape, in_dims, kNumberTypeInt8);
  ref_tensor(&w, w_shape, w_dims, kNumberTypeInt8);
  w.format_ = Format_KHWC;
  ref_tensor(&out, NULL, 0, kNumberTypeInt8);
  ConvParameter p;
  memset(&p, 0, sizeof(p));
  p.kernel_h_ = cp[0], p.kernel_w_ = cp[1], p.stride_h_ = cp[2], p.stride_w_ = cp[3];
  p.dilation_h_ = cp[4], p.dilation_w_ = cp[5], p.pad_mode_ = (PadType)cp[6];
  p.pad_u_ = cp[7], p.pad_d_ = cp[8], p.pad_l_ = cp[9], p.pad_r_ = cp[10], p.group_ = cp[11];
  const TensorC *ins[2] = {&in, &w};
  TensorC *outs[1] = {&out};
  int ret = Conv2dInferShape(ins, 2, outs, 1, (OpParameter *)&p);
  cp[0] = p.kernel_h_, cp[1] = p.kernel_w_, cp[7] = p.pad_u_, cp[8] = p.pad_d_, cp[9] = p.pad_l_, cp[10] = p.pad_r_;
  cp[11] = p.group_;
  return ref_emit_shape(ret, &out, out_shape, out_dims);
}

int ref_nnacl_infer_invalid(void) { return NNACL_INFER_INVALID; }
