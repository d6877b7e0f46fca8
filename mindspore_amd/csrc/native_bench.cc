// Native host for the launch-latency-sensitive parts of the benchmark: a C++ caller of the C ABI, which is what a
// MindSpore Lite provider kernel is.  (A Python caller spends about as long per call as a decode GEMV runs, so it
// measures the interpreter, not the kernel.)  Prints one JSON object.
//   native_bench decode <rows> <layers> <steps> <warmup>   the five 7B-class layer matrices x layers, cycled
//   native_bench warm <rows> <steps> <warmup>              each of the five matrices alone, back to back (its weights
//                                                          stay in the 256 MB Infinity Cache between launches)
//   native_bench read <mib> <steps> <warmup>               the library's plain read stream over slices of 3 GiB
//   native_bench bert <steps> <warmup>                     the four dynamic-quant MatMuls of a BERT-base layer at 4096
//                                                          rows (fp32 out), each launched back to back
//   native_bench dynmm <rows> <n> <k> <steps> <warmup>     one dynamic-quant MatMul shape
//   native_bench gemm <rows> <n> <k> <steps> <warmup>      one full-quant MatMul shape (int8 out)
//   native_bench dw <h> <w> <c> <steps> <warmup>           a 3x3 stride-1 depthwise convolution (ReLU6)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/mi355x_diag.h"
#include "../../include/mi355x_int8.h"

#define CHECK_HIP(x)                                                          \
  do {                                                                        \
    hipError_t e_ = (x);                                                      \
    if (e_ != hipSuccess) {                                                   \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                 \
      return 1;                                                               \
    }                                                                         \
  } while (0)
#define CHECK_MI(x)                                                           \
  do {                                                                        \
    int rc_ = (x);                                                            \
    if (rc_ != MI_OK) {                                                       \
      fprintf(stderr, "%s failed: %d (%s)\n", #x, rc_, mi_last_error());      \
      return 1;                                                               \
    }                                                                         \
  } while (0)

namespace {
struct Rng {  // SplitMix64
  uint64_t s;
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
};

// weights ~ clip(round(N(0,1) * 32), +-127): sum of 12 uniforms as the normal
int8_t normal_weight(Rng *r) {
  double acc = -6.0;
  const uint64_t a = r->next(), b = r->next();
  for (int i = 0; i < 6; ++i) acc += (double)((a >> (10 * i)) & 1023) / 1024.0;
  for (int i = 0; i < 6; ++i) acc += (double)((b >> (10 * i)) & 1023) / 1024.0;
  double v = std::round(acc * 32.0);
  v = v > 127 ? 127 : (v < -127 ? -127 : v);
  return (int8_t)v;
}

struct Shape {
  const char *name;
  int n, k;
};
const Shape kDecode[5] = {{"qkv", 12288, 4096}, {"o", 4096, 4096}, {"gate", 11008, 4096}, {"up", 11008, 4096},
                          {"down", 4096, 11008}};
}  // namespace

struct Matrix {
  mi_matmul *h = nullptr;
  int8_t *act = nullptr, *out = nullptr;
  int n = 0, k = 0;
  double bytes = 0;
};

static int make_matrix(const Shape &shape, int rows, Rng *rng, Matrix *m) {
  const int n = shape.n, k = shape.k;
  std::vector<int8_t> w((size_t)n * k);
  for (auto &x : w) x = normal_weight(rng);
  std::vector<double> scales(n);
  std::vector<int32_t> zps(n, 0), bias(n);
  for (int c = 0; c < n; ++c) {
    scales[c] = 0.001 + 0.009 * rng->uniform();
    bias[c] = (int32_t)(rng->next() % 10001) - 5000;
  }
  mi_matmul_desc d{};
  d.deep = k;
  d.col = n;
  d.b_transpose = 1;
  d.act_type = MI_ACT_NONE;
  d.in_scale = 0.02;
  d.in_zp = (int32_t)(rng->next() % 17) - 8;
  d.out_scale = 0.02 * 0.0055 * std::sqrt((double)k) * 40.0;
  d.out_zp = 0;
  d.filter_quant_num = n;
  d.filter_scales = scales.data();
  d.filter_zps = zps.data();
  // NATIVE_BENCH_NO_DECODE_PACK=1: handles without the blocked weight copy (2 rows and more then run on the GEMM tiles)
  if (getenv("NATIVE_BENCH_NO_DECODE_PACK") != nullptr) d.flags |= MI_MATMUL_NO_DECODE_PACK;
  CHECK_MI(mi_matmul_create(&d, w.data(), bias.data(), &m->h));
  std::vector<int8_t> a((size_t)rows * k);
  for (auto &x : a) x = (int8_t)(rng->next() & 0xff);
  CHECK_HIP(hipMalloc(&m->act, a.size()));
  CHECK_HIP(hipMalloc(&m->out, (size_t)rows * n));
  CHECK_HIP(hipMemcpy(m->act, a.data(), a.size(), hipMemcpyHostToDevice));
  m->n = n;
  m->k = k;
  m->bytes = (double)n * k + (double)rows * k + (double)rows * n + 16.0 * n;
  return 0;
}

static int run_warm(int rows, int steps, int warmup) {
  Rng rng{777};
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  printf("{\"mode\": \"warm\", \"m\": %d", rows);
  for (int s = 0; s < 5; ++s) {
    if (s == 3) continue;  // "up" has the shape of "gate"
    Matrix m;
    if (make_matrix(kDecode[s], rows, &rng, &m)) return 1;
    for (int i = 0; i < warmup; ++i) CHECK_MI(mi_matmul_run(m.h, m.act, rows, m.out, st));
    CHECK_HIP(hipStreamSynchronize(st));
    CHECK_HIP(hipEventRecord(e0, st));
    for (int i = 0; i < steps; ++i) CHECK_MI(mi_matmul_run(m.h, m.act, rows, m.out, st));
    CHECK_HIP(hipEventRecord(e1, st));
    CHECK_HIP(hipEventSynchronize(e1));
    float ms = 0;
    CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
    printf(", \"%s\": {\"n\": %d, \"k\": %d, \"us\": %.3f, \"gbps\": %.1f}", kDecode[s].name, m.n, m.k,
           ms / steps * 1e3, m.bytes / (ms / steps * 1e-3) / 1e9);
    mi_matmul_destroy(m.h);
    CHECK_HIP(hipFree(m.act));
    CHECK_HIP(hipFree(m.out));
  }
  printf("}\n");
  return 0;
}

static int run_decode(int rows, int layers, int steps, int warmup) {
  std::vector<mi_matmul *> handles;
  std::vector<int8_t *> acts, outs;
  double bytes = 0;
  Rng rng{12345};
  for (int l = 0; l < layers; ++l) {
    for (int s = 0; s < 5; ++s) {
      Matrix m;
      if (make_matrix(kDecode[s], rows, &rng, &m)) return 1;
      handles.push_back(m.h);
      acts.push_back(m.act);
      outs.push_back(m.out);
      bytes += m.bytes;
    }
  }
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  // gate and up read the same activation: they go out through mi_matmul_run_group (one launch), as a provider
  // would run sibling FullConnection nodes; NATIVE_BENCH_NO_GROUP=1 runs them one by one
  const bool group = getenv("NATIVE_BENCH_NO_GROUP") == nullptr;
  size_t launches = 0;
  auto step = [&]() -> int {
    launches = 0;
    for (size_t i = 0; i < handles.size(); ++i, ++launches) {
      if (group && i % 5 == 2) {
        mi_matmul *pair[2] = {handles[i], handles[i + 1]};
        int8_t *out[2] = {outs[i], outs[i + 1]};
        CHECK_MI(mi_matmul_run_group(pair, 2, acts[i], rows, out, st));
        ++i;
      } else {
        CHECK_MI(mi_matmul_run(handles[i], acts[i], rows, outs[i], st));
      }
    }
    return 0;
  };
  if (group) bytes -= (double)layers * rows * kDecode[3].k;  // the pair reads its activation rows once
  for (int i = 0; i < warmup; ++i)
    if (step()) return 1;
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i)
    if (step()) return 1;
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms = 0;
  CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
  const double ms_step = ms / steps;
  printf("{\"mode\": \"decode\", \"m\": %d, \"launches_per_step\": %zu, \"ms_per_step\": %.6f, \"us_per_launch\": %.3f, "
         "\"bytes_per_step\": %.0f, \"gbps\": %.1f}\n",
         rows, launches, ms_step, ms_step * 1e3 / launches, bytes, bytes / (ms_step * 1e-3) / 1e9);
  for (auto *h : handles) mi_matmul_destroy(h);
  return 0;
}

// one shape, enough distinct copies that the memory-side cache cannot hold them, launched round robin
static int run_shape(int n, int k, int rows, int steps, int warmup) {
  const Shape sh{"shape", n, k};
  const int copies = (int)(700e6 / ((double)n * k)) + 1;
  std::vector<Matrix> ms(copies);
  Rng rng{4242};
  for (auto &m : ms)
    if (make_matrix(sh, rows, &rng, &m)) return 1;
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  for (int i = 0; i < warmup * copies; ++i) CHECK_MI(mi_matmul_run(ms[i % copies].h, ms[i % copies].act, rows, ms[i % copies].out, st));
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps * copies; ++i) CHECK_MI(mi_matmul_run(ms[i % copies].h, ms[i % copies].act, rows, ms[i % copies].out, st));
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms_total = 0;
  CHECK_HIP(hipEventElapsedTime(&ms_total, e0, e1));
  const double us = ms_total * 1e3 / (steps * copies);
  printf("{\"mode\": \"shape\", \"n\": %d, \"k\": %d, \"m\": %d, \"copies\": %d, \"us\": %.3f, \"gbps\": %.1f}\n", n, k, rows, copies, us,
         ms[0].bytes / (us * 1e-6) / 1e9);
  for (auto &m : ms) mi_matmul_destroy(m.h);
  return 0;
}

static int run_read(int mib, int steps, int warmup) {
  const size_t total = (size_t)3 << 30, slice = (size_t)mib << 20;
  const int nslices = (int)(total / slice);
  char *buf = nullptr;
  CHECK_HIP(hipMalloc(&buf, total));
  CHECK_HIP(hipMemset(buf, 1, total));
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  for (int i = 0; i < warmup; ++i) CHECK_MI(mi_diag_stream_read(buf + (size_t)(i % nslices) * slice, (int64_t)slice, st));
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i)
    CHECK_MI(mi_diag_stream_read(buf + (size_t)((i + warmup) % nslices) * slice, (int64_t)slice, st));
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms = 0;
  CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
  printf("{\"mode\": \"read\", \"bytes\": %zu, \"ms\": %.6f, \"gbps\": %.1f}\n", slice, ms / steps,
         (double)slice / (ms / steps * 1e-3) / 1e9);
  return 0;
}

// One dynamic-quant MatMul (fp32 output) launched back to back; prints its JSON fragment.
static int time_dynmm(const char *name, int rows, int n, int k, int steps, int warmup, hipStream_t st,
                      double *ops_sum, double *ms_sum) {
  Rng rng{(uint64_t)(1000 + n + 7 * k)};
  std::vector<int8_t> w((size_t)n * k);
  for (auto &x : w) x = (int8_t)((int)(rng.next() % 255) - 127);
  std::vector<double> scales(n);
  std::vector<int32_t> zps(n, 0);
  std::vector<float> bias(n);
  for (int c = 0; c < n; ++c) {
    scales[c] = 0.001 + 0.009 * rng.uniform();
    bias[c] = (float)(rng.uniform() - 0.5);
  }
  mi_dynmm_desc d{};
  d.deep = k;
  d.col = n;
  d.b_transpose = 1;
  d.act_type = MI_ACT_NONE;
  d.filter_quant_num = n;
  d.filter_scales = scales.data();
  d.filter_zps = zps.data();
  mi_dynmm *h = nullptr;
  CHECK_MI(mi_dynmm_create(&d, w.data(), bias.data(), &h));
  std::vector<int8_t> a((size_t)rows * k);
  for (auto &x : a) x = (int8_t)(rng.next() & 0xff);
  int8_t *a_dev = nullptr;
  float *c_dev = nullptr;
  CHECK_HIP(hipMalloc(&a_dev, a.size()));
  CHECK_HIP(hipMalloc(&c_dev, (size_t)rows * n * 4));
  CHECK_HIP(hipMemcpy(a_dev, a.data(), a.size(), hipMemcpyHostToDevice));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  auto run = [&]() -> int { return mi_dynmm_run(h, a_dev, rows, 0.031, -3, c_dev, st); };
  for (int i = 0; i < warmup; ++i) CHECK_MI(run());
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i) CHECK_MI(run());
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms = 0;
  CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
  const double us = ms / steps * 1e3, ops = 2.0 * rows * n * k;
  const double bytes = (double)rows * k + (double)n * k + 4.0 * rows * n + 12.0 * n;
  printf("\"%s\": {\"rows\": %d, \"n\": %d, \"k\": %d, \"us\": %.3f, \"tops\": %.1f, \"algorithmic_bytes\": %.0f, "
         "\"gbps\": %.1f}",
         name, rows, n, k, us, ops / (us * 1e-6) / 1e12, bytes, bytes / (us * 1e-6) / 1e9);
  *ops_sum += ops;
  *ms_sum += ms / steps;
  mi_dynmm_destroy(h);
  CHECK_HIP(hipFree(a_dev));
  CHECK_HIP(hipFree(c_dev));
  return 0;
}

static int run_bert(int steps, int warmup) {
  const Shape shapes[4] = {{"qkv", 2304, 768}, {"out", 768, 768}, {"ffn1", 3072, 768}, {"ffn2", 768, 3072}};
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  double ops = 0, ms = 0;
  printf("{\"mode\": \"bert\", \"rows\": 4096, ");
  for (const Shape &s : shapes) {
    if (time_dynmm(s.name, 4096, s.n, s.k, steps, warmup, st, &ops, &ms)) return 1;
    printf(", ");
  }
  printf("\"total_us\": %.3f, \"total_tops\": %.1f}\n", ms * 1e3, ops / (ms * 1e-3) / 1e12);
  return 0;
}

static int run_dynmm(int rows, int n, int k, int steps, int warmup) {
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  double ops = 0, ms = 0;
  printf("{\"mode\": \"dynmm\", ");
  if (time_dynmm("shape", rows, n, k, steps, warmup, st, &ops, &ms)) return 1;
  printf("}\n");
  return 0;
}

// The decoder layer of run_decode as dynamic-quant MatMuls (int8 activations with a run-time scale, fp32 out): three
// layers' worth of distinct weights cycled, one launch per matrix.  no_pack = 1 creates the handles without the
// blocked weight copy, so that the same rows run on the GEMM tiles (what they did before the decode kernel had the
// fp32 epilogue).
static int run_dyndecode(int rows, int layers, int steps, int warmup, int no_pack) {
  struct DynMatrix {
    mi_dynmm *h;
    int8_t *act;
    float *out;
  };
  std::vector<DynMatrix> ms;
  double bytes = 0;
  Rng rng{4321};
  for (int l = 0; l < layers; ++l) {
    for (int s = 0; s < 5; ++s) {
      const int n = kDecode[s].n, k = kDecode[s].k;
      std::vector<int8_t> w((size_t)n * k);
      for (auto &x : w) x = normal_weight(&rng);
      std::vector<double> scales(n);
      std::vector<int32_t> zps(n, 0);
      for (int c = 0; c < n; ++c) scales[c] = 0.001 + 0.009 * rng.uniform();
      mi_dynmm_desc d{};
      d.deep = k;
      d.col = n;
      d.b_transpose = 1;
      d.act_type = MI_ACT_NONE;
      d.filter_quant_num = n;
      d.filter_scales = scales.data();
      d.filter_zps = zps.data();
      d.flags = no_pack ? MI_DYNMM_NO_DECODE_PACK : 0;
      DynMatrix m{};
      CHECK_MI(mi_dynmm_create(&d, w.data(), nullptr, &m.h));
      std::vector<int8_t> a((size_t)rows * k);
      for (auto &x : a) x = (int8_t)(rng.next() & 0xff);
      CHECK_HIP(hipMalloc(&m.act, a.size()));
      CHECK_HIP(hipMalloc(&m.out, (size_t)rows * n * 4));
      CHECK_HIP(hipMemcpy(m.act, a.data(), a.size(), hipMemcpyHostToDevice));
      ms.push_back(m);
      bytes += (double)n * k + (double)rows * k + 4.0 * rows * n + 12.0 * n;
    }
  }
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  // gate and up read the same activation: one launch through mi_dynmm_run_group, as the provider runs sibling
  // dynamic MatMuls (rows up to 32, handles with the blocked copy); NATIVE_BENCH_NO_GROUP=1 runs them one by one
  const bool group = getenv("NATIVE_BENCH_NO_GROUP") == nullptr && rows <= 32 && (rows == 1 || !no_pack);
  size_t launches = 0;
  auto step = [&]() -> int {
    launches = 0;
    for (size_t i = 0; i < ms.size(); ++i, ++launches) {
      if (group && i % 5 == 2) {
        mi_dynmm *pair[2] = {ms[i].h, ms[i + 1].h};
        float *out[2] = {ms[i].out, ms[i + 1].out};
        CHECK_MI(mi_dynmm_run_group(pair, 2, ms[i].act, rows, 0.031, -3, nullptr, 0, out, st));
        ++i;
      } else {
        CHECK_MI(mi_dynmm_run(ms[i].h, ms[i].act, rows, 0.031, -3, ms[i].out, st));
      }
    }
    return 0;
  };
  if (group) bytes -= (double)layers * rows * kDecode[3].k;  // the pair reads its activation rows once
  for (int i = 0; i < warmup; ++i)
    if (step()) return 1;
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i)
    if (step()) return 1;
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float t = 0;
  CHECK_HIP(hipEventElapsedTime(&t, e0, e1));
  const double ms_step = t / steps;
  printf("{\"mode\": \"dyndecode\", \"m\": %d, \"blocked_copy\": %d, \"launches_per_step\": %zu, \"ms_per_step\": %.6f, "
         "\"us_per_launch\": %.3f, \"bytes_per_step\": %.0f, \"gbps\": %.1f}\n",
         rows, no_pack ? 0 : 1, launches, ms_step, ms_step * 1e3 / launches, bytes, bytes / (ms_step * 1e-3) / 1e9);
  for (auto &m : ms) mi_dynmm_destroy(m.h);
  return 0;
}

static int run_gemm(int rows, int n, int k, int steps, int warmup) {
  const Shape sh{"gemm", n, k};
  Matrix m;
  Rng rng{99};
  if (make_matrix(sh, rows, &rng, &m)) return 1;
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  for (int i = 0; i < warmup; ++i) CHECK_MI(mi_matmul_run(m.h, m.act, rows, m.out, st));
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i) CHECK_MI(mi_matmul_run(m.h, m.act, rows, m.out, st));
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms = 0;
  CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
  const double us = ms / steps * 1e3;
  printf("{\"mode\": \"gemm\", \"rows\": %d, \"n\": %d, \"k\": %d, \"us\": %.3f, \"tops\": %.1f}\n", rows, n, k, us,
         2.0 * rows * n * k / (us * 1e-6) / 1e12);
  mi_matmul_destroy(m.h);
  return 0;
}

static int run_dw(int ih, int iw, int c, int steps, int warmup) {
  Rng rng{31};
  std::vector<int8_t> w((size_t)c * 9), x((size_t)ih * iw * c);
  for (auto &v : w) v = (int8_t)((int)(rng.next() % 255) - 127);
  for (auto &v : x) v = (int8_t)(rng.next() & 0xff);
  std::vector<double> scales(c);
  std::vector<int32_t> zps(c, 0), bias(c);
  for (int i = 0; i < c; ++i) {
    scales[i] = 0.001 + 0.009 * rng.uniform();
    bias[i] = (int32_t)(rng.next() % 4001) - 2000;
  }
  mi_conv_desc d{};
  d.in_channel = d.out_channel = d.group = c;
  d.kernel_h = d.kernel_w = 3;
  d.stride_h = d.stride_w = d.dilation_h = d.dilation_w = 1;
  d.pad_u = d.pad_d = d.pad_l = d.pad_r = 1;
  d.act_type = MI_ACT_RELU6;
  d.in_scale = 6.0 / 140.0;
  d.in_zp = -11;
  d.out_scale = 6.0 / 140.0;
  d.out_zp = 9;
  d.filter_quant_num = c;
  d.filter_scales = scales.data();
  d.filter_zps = zps.data();
  mi_conv *h = nullptr;
  CHECK_MI(mi_conv_create(&d, w.data(), bias.data(), &h));
  int8_t *in_dev = nullptr, *out_dev = nullptr;
  CHECK_HIP(hipMalloc(&in_dev, x.size()));
  CHECK_HIP(hipMalloc(&out_dev, x.size()));
  CHECK_HIP(hipMemcpy(in_dev, x.data(), x.size(), hipMemcpyHostToDevice));
  hipStream_t st;
  CHECK_HIP(hipStreamCreate(&st));
  hipEvent_t e0, e1;
  CHECK_HIP(hipEventCreate(&e0));
  CHECK_HIP(hipEventCreate(&e1));
  for (int i = 0; i < warmup; ++i) CHECK_MI(mi_conv_run(h, in_dev, 1, ih, iw, out_dev, st));
  CHECK_HIP(hipStreamSynchronize(st));
  CHECK_HIP(hipEventRecord(e0, st));
  for (int i = 0; i < steps; ++i) CHECK_MI(mi_conv_run(h, in_dev, 1, ih, iw, out_dev, st));
  CHECK_HIP(hipEventRecord(e1, st));
  CHECK_HIP(hipEventSynchronize(e1));
  float ms = 0;
  CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
  const double us = ms / steps * 1e3, bytes = 2.0 * x.size() + w.size();
  printf("{\"mode\": \"dw\", \"h\": %d, \"w\": %d, \"c\": %d, \"us\": %.3f, \"algorithmic_bytes\": %.0f, \"gbps\": %.1f}\n", ih,
         iw, c, us, bytes, bytes / (us * 1e-6) / 1e9);
  mi_conv_destroy(h);
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: native_bench decode <rows> <layers> <steps> <warmup> | warm <rows> <steps> <warmup> | read <mib> <steps> <warmup> | shape <n> <k> <rows> <steps> <warmup> | dyndecode <rows> <layers> <steps> <warmup> [no_pack] | bert <steps> <warmup> | dynmm <rows> <n> <k> <steps> <warmup> | gemm <rows> <n> <k> <steps> <warmup> | dw <h> <w> <c> <steps> <warmup>\n");
    return 2;
  }
  CHECK_MI(mi_init(0));
  if (strcmp(argv[1], "shape") == 0 && argc >= 7) return run_shape(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), atoi(argv[6]));
  if (strcmp(argv[1], "decode") == 0 && argc >= 6) return run_decode(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]));
  if (strcmp(argv[1], "warm") == 0 && argc >= 5) return run_warm(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]));
  if (strcmp(argv[1], "dyndecode") == 0 && argc >= 6)
    return run_dyndecode(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), argc >= 7 ? atoi(argv[6]) : 0);
  if (strcmp(argv[1], "bert") == 0 && argc >= 4) return run_bert(atoi(argv[2]), atoi(argv[3]));
  if (strcmp(argv[1], "dynmm") == 0 && argc >= 7) return run_dynmm(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), atoi(argv[6]));
  if (strcmp(argv[1], "gemm") == 0 && argc >= 7) return run_gemm(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), atoi(argv[6]));
  if (strcmp(argv[1], "dw") == 0 && argc >= 7) return run_dw(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]), atoi(argv[5]), atoi(argv[6]));
  if (strcmp(argv[1], "read") == 0 && argc >= 5) return run_read(atoi(argv[2]), atoi(argv[3]), atoi(argv[4]));
  fprintf(stderr, "bad arguments\n");
  return 2;
}
