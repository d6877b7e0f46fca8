// Internal declarations shared by the HIP translation units of libmi355x_int8.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi355x_int8.h"

namespace mi {

void set_error(const char *fmt, ...);

#define MI_HIP_CHECK(expr)                                                                   \
  do {                                                                                       \
    hipError_t _e = (expr);                                                                  \
    if (_e != hipSuccess) {                                                                  \
      mi::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
      return MI_ERROR;                                                                       \
    }                                                                                        \
  } while (0)

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }
inline int64_t round_up64(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// Weight rows (output channels) and the contraction dimension are padded so that no kernel needs bounds checks on
// the weight operand: rows to a multiple of kNPad, K to a multiple of kKPad (bytes, two 128-byte GEMM steps), zero filled.
constexpr int kNPad = 256;
constexpr int kKPad = 256;

// The value the 256 x 256 GEMM tile's accumulators start from (taken out again in the epilogue); the host's proof that
// the cheap rounding form cannot overflow includes it.
constexpr uint32_t kAccBias = 0x2AAAAAAAu;

// ---- int8 requantising epilogue parameters (device arrays are padded to kNPad entries) ----
struct RequantParams {
  const int32_t *mult;    // 31-bit mantissa per channel
  const int32_t *bias2;   // K*zx*zw - zx*sum(w) + bias
  const int32_t *rshift;  // e = -right_shift clamped to [0, 31]
  const int32_t *lshift;  // left shift (generic path only)
  const int32_t *zw;      // weight zero point per channel (HAS_ZW only)
  int32_t zo, amin, amax;
  int has_zw;  // any weight zero point is non-zero -> input row sums are needed
  int fast;    // host proved: all lshift == 0, 1 <= e <= 30, no mult == INT32_MIN, amin <= amax, and none of
               // acc + bias2, srdhm + 2^(e-1) + (zo << e) can overflow int32
  // Single-multiply form of the cheap rounding, for accumulators that start from kAccBias (gemm_i8.hip).  With
  // a = accumulator register read as unsigned (true sum + kAccBias [- rowsum * zw]):
  //   x = high dword of (a * mult2 + c2)      == floor(((sum + bias2) * mult + 2^30) / 2^31), the doubling high mul
  //   y = clamp((x + pre + [x >= 0]) >> e)    pre = 2^(e-1) + (zo << e) - 1; [x >= 0] is the carry of a * mult2 + c2
  // mult2 = 2 * mult, c2 = 2 * (bias2 - kAccBias) * mult + 2^31 (mod 2^64, negative as a signed number), in dwords.
  const uint32_t *mult2;
  const uint32_t *c2lo, *c2hi;
  const int32_t *pre;
  int fast2;   // fast, and every mult >= 0, every c2 < 0, and K * 16384 + K * 128 * |zw| <= kAccBias (a in [0, 2^31))
};

// ---- fp32 dequantising epilogue (dynamic-quant MatMul) ----
struct DequantParams {
  const float *wscale;           // (float)filter_scale per channel (padded; per-tensor is broadcast at Prepare)
  const float *bias;             // fp32 bias or nullptr
  const int32_t *wsum;           // sum_k w[n][k]
  const mi_dq_params *qp_dev;    // input scale / zero point on the device, or nullptr -> use sx / zx below
  float sx;
  int32_t zx;
  int32_t zw0;
  int32_t deep;  // true K
  int32_t act;
  int32_t per_row;  // input scale of row r is qp_dev[r].scale_f; the zero point is qp_dev[0].zero_point
};

// Packed weights: n_pad rows (output channels) of k_pad contraction bytes, zero filled past K, with row stride ldw.
// The stride is skewed to an odd multiple of 256 bytes: the kernels fetch 16 rows x 64 bytes per wave instruction,
// and with a power-of-two stride those 16 requests would all fall into the same memory channel.
struct WeightView {
  const int8_t *w;
  int k_pad;
  int ldw;
  // Second copy for the matrix-core decode kernel (2..64 activation rows), or nullptr: the same bytes regrouped into
  // 1 KiB blocks [row / 16][k / 64], the 64 16-byte chunks of a block in the order the lanes of the MFMA operand take
  // them ([(k % 64) / 16][row % 16]), so that a wave instruction fetches 1 KiB front to back.  Built on the device
  // when the handle is created (launch_block_weights).
  const int8_t *blocked;
};
inline int weight_row_stride(int k_pad) { return (k_pad / 256) % 2 == 0 ? k_pad + 256 : k_pad; }

// A: int8 activations [M][lda] (lda in bytes, multiple of 16, base 16-byte aligned, K % 16 == 0);
// W: packed weights (above); C: [M][ldc] elements with n % 4 == 0, ldc % 4 == 0 and a 4-byte (int8) /
// 16-byte (fp32) aligned base -- other output shapes go through a padded scratch buffer and launch_copy_rows.
int launch_gemm_requant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream);
int launch_gemm_dequant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const DequantParams &dq, float *c, int64_t ldc, hipStream_t stream);

// Skinny-M path (m <= kGemvMaxRows): streams the weights once with 16-byte coalesced loads.
constexpr int kGemvMaxRows = 64;
constexpr int kGemvGroupMaxRows = 32;  // the group launches (several matrices, one launch) stop here
// 65..128 rows keep the matrix-core decode kernel only where it has at most one workgroup per CU (16 channels each,
// so at most 4096 channels) and a reduction long enough to pay for its set-up.  Measured against the GEMM's
// weight-stream tiles at 128 rows, weights not cache-resident (us per launch): 4096 x 4096 14.5 against 22.6,
// 4096 x 11008 31.5 against 52.7, 1024 x 4096 12.7 against 22.5, 4096 x 1024 6.8 against 8.8, 2048 x 768 7.1 against
// 6.7; 6144 x 4096 25.0 against 22.9, 8192 x 4096 26.6 against 23.1.
constexpr int kGemvNarrowMaxRows = 128;
constexpr int kGemvNarrowChannels = 4096;  // at most this many
constexpr int kGemvNarrowMinK = 1024;      // padded reduction length from which those rows come here
inline bool gemv_takes_rows(int rows, int n, int k_pad) {
  return rows <= kGemvMaxRows || (rows <= kGemvNarrowMaxRows && n <= kGemvNarrowChannels && k_pad >= kGemvNarrowMinK);
}
constexpr int kGemvDotRows = 2;  // up to here the v_dot4 kernel can run (it does for one row, and for two when the handle has no blocked copy), above it the MFMA kernel
int launch_gemv_requant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const RequantParams &rq, int8_t *c, int64_t ldc, hipStream_t stream);

// 1..64 rows of the dynamic-quant MatMul (fp32 out) on the blocked weight copy (w.blocked must be there).
int launch_gemv_dequant(const int8_t *a, int64_t lda, int m, int k, const WeightView &w, int n,
                        const DequantParams &dq, float *c, int64_t ldc, hipStream_t stream);

// Up to four dynamic-quant MatMuls with the same K against the same activation rows, as one launch; member i writes
// c[i] (fp32) with row stride n[i].  For more than one row every member needs w.blocked.
int launch_gemv_group_dequant(const int8_t *a, int64_t lda, int m, int k, int count, const WeightView *w, const int *n,
                              const DequantParams *dq, float *const *c, hipStream_t stream);

// Up to four weight matrices with the same K against the same activation rows, as one launch (the grid is the
// concatenation of the members' grids); member i writes c[i] with row stride n[i].
int launch_gemv_group(const int8_t *a, int64_t lda, int m, int k, int count, const WeightView *w, const int *n,
                      const RequantParams *rq, int8_t *const *c, hipStream_t stream);

// Per-device set-up of the skinny-M kernels (function attributes); called by mi_init with the device current.
int gemv_prepare_device();

// Regroups packed row-major weights into the blocked copy described at WeightView::blocked.
int launch_block_weights(const int8_t *w, int n_pad, int k_pad, int ldw, int8_t *blocked, hipStream_t stream);

// Copies [rows][k] (row stride src_ld bytes) into a zero-padded [rows][k16] buffer, k16 = round_up(k, 16).
int launch_pad_rows(const int8_t *src, int64_t src_ld, int rows, int k, int8_t *dst, int k16, hipStream_t stream);

// dst[row][0..row_bytes) = src[row][0..row_bytes); strides in bytes.
int launch_copy_rows(const void *src, int64_t src_ld, int rows, int row_bytes, void *dst, int64_t dst_ld,
                     hipStream_t stream);

struct ConvGeom {
  int batch, in_h, in_w, in_c, out_h, out_w, out_c;
  int kernel_h, kernel_w, stride_h, stride_w, dilation_h, dilation_w, pad_u, pad_l;
};
// im2col into [batch*out_h*out_w][k16] with K order (kh, kw, ic); out-of-image taps are `fill`, the K tail is zero.
int launch_im2col(const int8_t *in, const ConvGeom &g, int fill, int8_t *dst, int k16, hipStream_t stream);
// Dense convolution with kernel_h * kernel_w * in_c <= 64 and out_c <= 128, out_c % 4 == 0, straight from the image
// (no im2col buffer); w: packed row-major weights with row stride ldw, K order (kh, kw, ic).
int launch_conv_smallk(const int8_t *in, const ConvGeom &g, int fill, int k_true, const int8_t *w, int ldw,
                       const RequantParams &rq, int8_t *out, hipStream_t stream);
// Depthwise conv + requantisation, weights pre-offset to int16 [KH*KW][C].  bias_folded = bias - zx8 * sum_t w16[t][c]
// (used by the channel-vectorised kernel, which reads out-of-image taps as zx8); rq.fast: the host proved the cheap
// rounding form exact for every channel.
int launch_conv_dw(const int8_t *in, const ConvGeom &g, const int16_t *w16, const int32_t *bias,
                   const int32_t *bias_folded, int zx8, const RequantParams &rq, int8_t *out, hipStream_t stream);

// The requantising GEMM with its activation operand gathered from an NHWC image (in_c % 16 == 0): the im2col
// convolution without the buffer.  fill16: 16 bytes of the value out-of-image taps take, in device memory.
bool gemm_conv_supported(const ConvGeom &g, const void *in, const void *out);
int launch_gemm_conv_requant(const int8_t *in, const ConvGeom &g, const int8_t *fill16, const WeightView &w,
                             const RequantParams &rq, int8_t *out, hipStream_t stream);

// DynamicQuant: per-block min/max partials, then quantise (every block re-reduces the partials).
constexpr int kDqMaxBlocks = 1024;
int launch_dynquant(const float *x, int64_t n, int symmetric, float2 *partials, mi_dq_params *params, int8_t *q,
                    hipStream_t stream);
// One {scale, zero point} per contiguous run of `unit` elements; params has `segments` entries.
int launch_dynquant_segments(const float *x, int64_t segments, int64_t unit, int symmetric, mi_dq_params *params,
                             int8_t *q, hipStream_t stream);

}  // namespace mi
