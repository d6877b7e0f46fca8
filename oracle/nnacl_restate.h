/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the arithmetic of MindSpore Lite's int8 hot path
 * (nnacl int8 kernels + the Lite CPU wrappers that drive them).  Nothing in the shipped library links,
 * loads or calls this file; it is the checker used by tests, the smoke entry and the CPU-baseline leg of
 * the benchmark.
 *
 * All functions are layout-free: row-major in, row-major out.  nnacl's packed layouts (4x16, 8x4 blocks)
 * are invisible in the results and are therefore not reproduced here.
 *
 * Reference paths are relative to the reference tree root:
 *   NN/ = mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/
 *   LK/ = mindspore/lite/src/litert/kernel/cpu/
 */
#ifndef ORACLE_NNACL_RESTATE_H_
#define ORACLE_NNACL_RESTATE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* activation types, numeric values of schema ActivationType (mindspore/lite/schema/ops_types.fbs:62-66) */
#define ORC_ACT_NONE 0
#define ORC_ACT_RELU 1
#define ORC_ACT_RELU6 3

/* ---- fixed point (NN/int8/fixed_point.c) ---- */
int32_t orc_srdhm(int32_t a, int32_t b);                                    /* :26-35 */
int32_t orc_rdiv_pot(int32_t x, int32_t exponent);                          /* :48-56 */
int32_t orc_mul_by_quant_mult(int32_t v, int32_t mult, int32_t ls, int32_t rs); /* :66-68 */

/* ---- quantize params (NN/int8/quantize.c) ---- */
void orc_quantize_multiplier(double m, int32_t *mult, int32_t *shift);      /* :113-161 */
void orc_round_param(double m, int32_t *mult, int32_t *ls, int32_t *rs);    /* :39-51 */
void orc_round_param_single(double m, int32_t *mult, int32_t *ls, int32_t *rs); /* :53-72 */
void orc_act_range(int relu, int relu6, int32_t zp, float scale, int32_t *mn, int32_t *mx); /* :76-94 */
/* LK/int8/matmul_base_int8.cc:235-273 and LK/base/convolution_base.cc:416-427 */
void orc_requant_params(double sx, const double *sw, int nfilt, double so, int32_t *mult, int32_t *ls, int32_t *rs);

/* ---- full-quant MatMul / FullConnection (LK/int8/matmul_base_int8.cc + NN/int8/matmul_int8.c:296-331) ---- */
int orc_matmul_int8(const int8_t *a, const int8_t *w, const int32_t *bias, int8_t *c, int m, int n, int k,
                    int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so,
                    int zo, int act_type);

/* ---- Conv2D int8, group 1 (1x1: LK/int8/convolution_1x1_int8.cc; other: LK/int8/convolution_int8.cc +
 *      NN/int8/conv_int8.c:758-913).  Weight [OC][KH][KW][IC], in/out NHWC. ---- */
typedef struct orc_conv_shape {
  int batch, in_h, in_w, in_c;
  int out_h, out_w, out_c;
  int kernel_h, kernel_w, stride_h, stride_w, dilation_h, dilation_w;
  int pad_u, pad_l;
} orc_conv_shape;

int orc_conv_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const orc_conv_shape *s,
                  double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo, int act_type);

/* ---- depthwise conv int8, per-tensor activations (LK/int8/convolution_depthwise_int8.cc +
 *      NN/int8/conv_depthwise_int8.c:24-140).  Weight memory [C][KH*KW]. ---- */
int orc_conv_dw_int8(const int8_t *in, const int8_t *w, const int32_t *bias, int8_t *out, const orc_conv_shape *s,
                     double sx, int zx, const double *sw, const int32_t *zw, int nfilt, double so, int zo,
                     int act_type);

/* ---- DynamicQuant (LK/int8/dynamic_quant.cc, NN/int8/dynamic_quant_int8.c, NN/int8/quant_dtype_cast_int8.c) ---- */
void orc_minmax_fp32(const float *x, int64_t n, float *mn, float *mx);       /* dynamic_quant_int8.c:19-27 */
void orc_dynquant_params(float mn, float mx, int symmetric, double *scale, int32_t *zp); /* dynamic_quant.cc:156-186 */
void orc_quantize_fp32_int8(const float *x, int8_t *q, float scale, int32_t zp, int64_t n); /* quant_dtype_cast_int8.c:180-203 */
int orc_dynamic_quant(const float *x, int64_t n, int symmetric, int8_t *q, double *scale, int32_t *zp);

/* ---- dynamic-quant MatMul (LK/int8/matmul_dynamic_int8.cc + NN/int8/dynamic_matmul_int8.c:99-143) ---- */
int orc_dynamic_quant_segments(const float *x, int64_t segments, int64_t unit, int symmetric, int8_t *q,
                               double *scales, int32_t *zps);
int orc_dynamic_matmul_rows(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                            int b_transpose, const float *sx_rows, int zx, const double *sw, const int32_t *zw,
                            int nfilt, int act_type);
int orc_dynamic_matmul(const int8_t *a, const int8_t *w, const float *bias, float *c, int m, int n, int k,
                       int b_transpose, double sx, int zx, const double *sw, const int32_t *zw, int nfilt,
                       int act_type);

/* number of OpenMP threads the loops above use (1 = scalar port) */
void orc_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
