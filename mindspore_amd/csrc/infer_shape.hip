// Shape inference for MatMulFusion, FullConnection and Conv2DFusion: what a provider's KernelInterface::Infer
// answers.  Pure host arithmetic (no device code in this file); results follow nnacl's inference functions
// (nnacl/infer/matmul_infer.c, full_connection_infer.c, conv2d_infer.c), including their corner cases.
#include <math.h>

#include "common.h"

namespace {

// A shape under construction: at most MI_MAX_DIMS extents.
struct Dims {
  int32_t v[MI_MAX_DIMS];
  int n;
  bool load(const int32_t *src, int count) {
    if (count < 0 || count > MI_MAX_DIMS || (count > 0 && src == nullptr)) return false;
    n = count;
    for (int i = 0; i < count; ++i) v[i] = src[i];
    return true;
  }
  bool push_front(int32_t x) {
    if (n >= MI_MAX_DIMS) return false;
    for (int i = n; i > 0; --i) v[i] = v[i - 1];
    v[0] = x;
    ++n;
    return true;
  }
  bool push_back(int32_t x) {
    if (n >= MI_MAX_DIMS) return false;
    v[n++] = x;
    return true;
  }
  void pop_front() {
    for (int i = 0; i + 1 < n; ++i) v[i] = v[i + 1];
    --n;
  }
  bool known() const {
    for (int i = 0; i < n; ++i)
      if (v[i] < 0) return false;
    return true;
  }
  int32_t &back(int from_end = 0) { return v[n - 1 - from_end]; }
};

int fail(const char *what) {
  mi::set_error("shape inference: %s", what);
  return MI_INFER_ERR;
}

int emit(const Dims &d, int32_t *out_shape, int32_t *out_dims) {
  for (int i = 0; i < d.n; ++i) out_shape[i] = d.v[i];
  *out_dims = d.n;
  return MI_OK;
}

}  // namespace

extern "C" int mi_infer_matmul(const int32_t *a_shape, int32_t a_dims, const int32_t *b_shape, int32_t b_dims,
                               const int32_t *bias_shape, int32_t bias_dims, int32_t transpose_a,
                               int32_t transpose_b, int32_t *out_shape, int32_t *out_dims) {
  if (out_shape == nullptr || out_dims == nullptr) {
    mi::set_error("mi_infer_matmul: null output");
    return MI_NULL_PTR;
  }
  Dims a, b, bias;
  if (!a.load(a_shape, a_dims) || !b.load(b_shape, b_dims) || !bias.load(bias_shape, bias_dims)) {
    return fail("bad rank or null shape");
  }
  if (!a.known() || !b.known() || !bias.known()) return MI_INFER_INVALID;
  // ranks are equalised first, so a vector only stays a vector when both operands are vectors
  Dims &shorter = a.n > b.n ? b : a;
  const int diff = a.n > b.n ? a.n - b.n : b.n - a.n;
  for (int i = 0; i < diff; ++i) shorter.push_front(1);
  // a bias of rank > 1 must be [1, ..., 1, N]
  for (int i = 0; i + 1 < bias.n; ++i)
    if (bias.v[i] != 1) return fail("bias has a leading extent other than 1");
  bool a_was_vector = false, b_was_vector = false;
  if (a.n == 1) {
    a.push_front(1);
    a_was_vector = true;
  }
  if (b.n == 1) {
    b.push_back(1);
    b_was_vector = true;
  }
  if (a.n < 2 || b.n < 2) return fail("an operand has no dimensions");
  const int lead = (a.n < b.n ? a.n : b.n) - 2;
  for (int i = 0; i < lead; ++i) {
    const int32_t lo = a.v[i] < b.v[i] ? a.v[i] : b.v[i], hi = a.v[i] < b.v[i] ? b.v[i] : a.v[i];
    if (lo != 0 && hi % lo != 0) return fail("leading extents do not broadcast");
  }
  if (transpose_a) {
    const int32_t t = a.back();
    a.back() = a.back(1);
    a.back(1) = t;
  }
  if (transpose_b) {
    const int32_t t = b.back();
    b.back() = b.back(1);
    b.back(1) = t;
  }
  if (bias.n == 1 && bias.v[0] != b.back()) return fail("bias length differs from the column count");
  if (a.back() != b.back(1)) return fail("contraction lengths differ");
  Dims c = a;
  c.back() = b.back();
  if (a_was_vector) c.pop_front();
  if (b_was_vector) --c.n;
  for (int i = 0; i < lead; ++i) c.v[i] = a.v[i] > b.v[i] ? a.v[i] : b.v[i];
  return emit(c, out_shape, out_dims);
}

extern "C" int mi_infer_fullconnection(const int32_t *a_shape, int32_t a_dims, const int32_t *w_shape, int32_t w_dims,
                                       const int32_t *bias_shape, int32_t bias_dims, int32_t has_bias,
                                       int32_t use_axis, int32_t axis, int32_t *out_shape, int32_t *out_dims) {
  if (out_shape == nullptr || out_dims == nullptr) {
    mi::set_error("mi_infer_fullconnection: null output");
    return MI_NULL_PTR;
  }
  Dims a, w, bias;
  if (!a.load(a_shape, a_dims) || !w.load(w_shape, w_dims) || !bias.load(bias_shape, bias_dims)) {
    return fail("bad rank or null shape");
  }
  if (!a.known() || !w.known() || !bias.known()) return MI_INFER_INVALID;
  if ((has_bias != 0) != (bias.n > 0)) return fail("has_bias disagrees with the inputs");
  if (use_axis && (axis < 1 || axis > a.n)) return fail("axis out of range");
  if (w.n < 2) return fail("weight is not [N, K]");
  int32_t k = 1;
  if (use_axis) {
    for (int i = axis; i < a.n; ++i) k = (int32_t)((uint32_t)k * (uint32_t)a.v[i]);
    if (k != w.v[1]) return fail("folded input length differs from K");
  } else {
    k = w.v[1];
  }
  if (has_bias && bias.v[0] != w.v[0]) return fail("bias length differs from N");
  Dims c = a;
  if (use_axis) {
    if (axis >= MI_MAX_DIMS) return fail("axis out of range");
    c.n = axis + 1;
    c.v[axis] = w.v[0];
  } else {
    int32_t total = 1;
    for (int i = 0; i < a.n; ++i) total = (int32_t)((uint32_t)total * (uint32_t)a.v[i]);
    if (k == 0) return fail("K is zero");
    c.n = 2;
    c.v[0] = total / k;
    c.v[1] = w.v[0];
  }
  return emit(c, out_shape, out_dims);
}

extern "C" int mi_infer_conv2d(const int32_t *in_shape, int32_t in_dims, const int32_t *w_shape, int32_t w_dims,
                               mi_conv_infer *p, int32_t *out_shape, int32_t *out_dims) {
  if (p == nullptr || out_shape == nullptr || out_dims == nullptr) {
    mi::set_error("mi_infer_conv2d: null argument");
    return MI_NULL_PTR;
  }
  Dims in, w;
  if (!in.load(in_shape, in_dims) || !w.load(w_shape, w_dims)) return fail("bad rank or null shape");
  if (w.n != 4) return fail("weight is not [OC, KH, KW, IC]");
  if (p->group == 0) p->group = w.v[0];
  if (!in.known() || !w.known()) return MI_INFER_INVALID;
  if (p->kernel_h == -1) p->kernel_h = w.v[1];
  if (p->kernel_w == -1) p->kernel_w = w.v[2];
  if (in.n == 0) return MI_INFER_INVALID;
  if (in.n != 4) return fail("input is not NHWC");
  const int32_t in_c = in.v[3], w_ic = w.v[3];
  // dense: in_c == w_ic; depthwise: w_ic == 1 is spelled "in_c == 1" by the reference; grouped: in_c / group == w_ic
  if (p->group == 0) return fail("group is zero");
  if (in_c != w_ic && in_c != 1 && in_c / p->group != w_ic) return fail("input channels do not fit the weight");
  if (w_ic == 0) return fail("weight has no input channels");
  if (p->group != 1 && p->group != in_c && p->group != in_c / w_ic) return fail("group does not fit the channels");
  if (p->stride_h <= 0 || p->stride_w <= 0) return fail("stride must be positive");
  if (p->kernel_h >= 10000 || p->kernel_w >= 10000) return fail("kernel too large");
  if (p->kernel_h != w.v[1] || p->kernel_w != w.v[2]) return fail("kernel size differs from the weight");

  const int32_t in_h = in.v[1], in_w = in.v[2];
  const int64_t span_h = (int64_t)p->kernel_h * p->dilation_h, span_w = (int64_t)p->kernel_w * p->dilation_w;
  if (span_h != (int32_t)span_h || span_w != (int32_t)span_w) return fail("dilated kernel overflows");
  int32_t out_h, out_w;
  if (p->pad_mode == MI_PAD_SAME) {
    out_w = (int32_t)ceil((float)in_w / (float)p->stride_w);
    out_h = (int32_t)ceil((float)in_h / (float)p->stride_h);
    const int32_t all_h = (out_h - 1) * p->stride_h + (p->kernel_h - 1) * p->dilation_h + 1 - in_h;
    const int32_t all_w = (out_w - 1) * p->stride_w + (p->kernel_w - 1) * p->dilation_w + 1 - in_w;
    p->pad_u = all_h < 0 ? 0 : all_h / 2;
    p->pad_d = all_h < 0 ? 0 : all_h - p->pad_u;
    p->pad_l = all_w < 0 ? 0 : all_w / 2;
    p->pad_r = all_w < 0 ? 0 : all_w - p->pad_l;
  } else if (p->pad_mode == MI_PAD_VALID) {
    // single-precision steps in the reference's order: ((in + pad + pad) - (k - 1) * d) / stride, then ceil
    const float num_w = (float)in_w + (float)p->pad_l + (float)p->pad_r - ((float)p->kernel_w - 1) * (float)p->dilation_w;
    const float num_h = (float)in_h + (float)p->pad_u + (float)p->pad_d - ((float)p->kernel_h - 1) * (float)p->dilation_h;
    out_w = (int32_t)ceil(num_w / (float)p->stride_w);
    out_h = (int32_t)ceil(num_h / (float)p->stride_h);
  } else {
    const int32_t ext_w = (p->kernel_w - 1) * p->dilation_w + 1, ext_h = (p->kernel_h - 1) * p->dilation_h + 1;
    out_w = (in_w + p->pad_l + p->pad_r - ext_w) / p->stride_w + 1;
    out_h = (in_h + p->pad_u + p->pad_d - ext_h) / p->stride_h + 1;
  }
  if (p->kernel_h > in_h + p->pad_u + p->pad_d || p->kernel_w > in_w + p->pad_l + p->pad_r) {
    return fail("kernel larger than the padded input");
  }
  Dims c;
  c.n = 4;
  c.v[0] = in.v[0];
  c.v[1] = out_h >= 0 ? out_h : 1;
  c.v[2] = out_w >= 0 ? out_w : 1;
  c.v[3] = w.v[0];
  return emit(c, out_shape, out_dims);
}

// The batch broadcast of MatMul operands (InitBroadcastParams, mindspore/lite/src/litert/kernel/cpu/fp32/
// matmul_fp32_base.cc:576-646): both shapes are brought to the same rank (at least 4) with leading ones; a batch
// extent of one operand may be smaller than the other's when it divides it, and output matrix i then takes the
// operand's matrix at the proportionally scaled index.
extern "C" int mi_matmul_broadcast_offsets(const int32_t *a_shape, int32_t a_dims, const int32_t *b_shape,
                                           int32_t b_dims, int32_t capacity, int32_t *batch, int32_t *a_offsets,
                                           int32_t *b_offsets) {
  if (batch == nullptr || a_offsets == nullptr || b_offsets == nullptr) {
    mi::set_error("mi_matmul_broadcast_offsets: null output");
    return MI_NULL_PTR;
  }
  Dims a, b;
  if (!a.load(a_shape, a_dims) || !b.load(b_shape, b_dims) || a.n < 2 || b.n < 2 || !a.known() || !b.known()) {
    mi::set_error("mi_matmul_broadcast_offsets: operands must have rank 2..%d and known extents", MI_MAX_DIMS);
    return MI_PARAM_INVALID;
  }
  const int rank = a.n > b.n ? (a.n > 4 ? a.n : 4) : (b.n > 4 ? b.n : 4);
  if (rank > MI_MAX_DIMS) return MI_PARAM_INVALID;
  while (a.n < rank) a.push_front(1);
  while (b.n < rank) b.push_front(1);
  const int nb = rank - 2;  // batch axes
  int64_t sizes[MI_MAX_DIMS] = {0}, a_sizes[MI_MAX_DIMS] = {0}, b_sizes[MI_MAX_DIMS] = {0};  // products from axis j to the last batch axis
  int64_t out_batch = 1;
  for (int j = nb - 1; j >= 0; --j) {
    const int64_t mx = a.v[j] > b.v[j] ? a.v[j] : b.v[j];
    const int64_t mn_raw = a.v[j] < b.v[j] ? a.v[j] : b.v[j];
    const int64_t mn = mn_raw > 0 ? mn_raw : 1;
    if (mx != mn && mx % mn != 0) {
      mi::set_error("mi_matmul_broadcast_offsets: batch extents %d and %d cannot be broadcast", a.v[j], b.v[j]);
      return MI_PARAM_INVALID;
    }
    sizes[j] = (j == nb - 1 ? 1 : sizes[j + 1]) * mx;
    a_sizes[j] = (j == nb - 1 ? 1 : a_sizes[j + 1]) * a.v[j];
    b_sizes[j] = (j == nb - 1 ? 1 : b_sizes[j + 1]) * b.v[j];
    out_batch *= mx;
  }
  if (out_batch > capacity || out_batch <= 0) {
    mi::set_error("mi_matmul_broadcast_offsets: %lld output matrices, room for %d", (long long)out_batch, capacity);
    return MI_PARAM_INVALID;
  }
  *batch = (int32_t)out_batch;
  for (int64_t i = 0; i < out_batch; ++i) {
    int64_t delta = i, ao = 0, bo = 0;
    for (int j = 0; j < nb; ++j) {
      if (j > 0) delta %= sizes[j];
      const int64_t mx = a.v[j] > b.v[j] ? a.v[j] : b.v[j];
      if (j < nb - 1) {
        ao += (delta / sizes[j + 1] * a.v[j] / mx) * a_sizes[j + 1];
        bo += (delta / sizes[j + 1] * b.v[j] / mx) * b_sizes[j + 1];
      } else {
        ao += delta * a.v[j] / mx;
        bo += delta * b.v[j] / mx;
      }
    }
    a_offsets[i] = (int32_t)ao;
    b_offsets[i] = (int32_t)bo;
  }
  return MI_OK;
}
