// C ABI of libmi355x_int8.so: handle objects that own packed weights, derived quant parameters and workspaces on
// the device, and route each Run to the right kernel.  Everything the Lite CPU wrappers do at Prepare()/ReSize()
// time happens in mi_*_create on the host with strict IEEE arithmetic (this file is compiled with
// -ffp-contract=off); the device only ever sees integers and already-rounded floats.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <memory>
#include <new>
#include <vector>

#include "common.h"
#include "quant_math.h"

namespace mi {

static thread_local char g_err[512] = "";
static int g_device = -1;
// how often the library made the host wait for a stream (mi_debug_sync_count): the copies with host tensors, the
// parameter fetch of DynamicQuant, mi_stream_synchronize
static std::atomic<int64_t> g_sync_count{0};
static hipError_t counted_sync(hipStream_t s) {
  g_sync_count.fetch_add(1, std::memory_order_relaxed);
  return hipStreamSynchronize(s);
}

// Scratch memory of mi_matmul_run_noalloc: static device memory, so the entry point never allocates.  Every GPU the
// library is initialised on holds its own copy of the array at its own address; the array's name is only a host-side
// stand-in, so host code uses the per-device address that mi_init looked up (g_scratch_ptr), never the name.
constexpr size_t kScratchBytes = MI_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices] = {};

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

static int ensure_device() {
  if (g_device < 0) {
    set_error("mi_init has not been called (or found no gfx950 device)");
    return MI_ERROR;
  }
  MI_HIP_CHECK(hipSetDevice(g_device));
  return MI_OK;
}

// ---- host-side quant parameter derivation -----------------------------------------------------------------------
// QuantizeMultiplier (reference nnacl/int8/quantize.c:113-161): |m| = q * 2^shift, q in [0.5, 1);
// mult = round_half_up(q * 2^31) with the carry renormalised; the sign moves onto mult.
static void quantize_multiplier(double m, int32_t *mult, int32_t *shift) {
  if (m == 0.0 || m != m) {
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
  const double q = frexp(fabs(m), &e);
  uint64_t sig = (uint64_t)ldexp(q, 53);
  uint64_t r = ((sig >> 21) + 1u) >> 1;
  if (r == ((uint64_t)1 << 31)) {
    r >>= 1;
    ++e;
  }
  *shift = e;
  *mult = m < 0 ? -(int32_t)r : (int32_t)r;
}

static void round_param(double m, int32_t *mult, int32_t *ls, int32_t *rs) {
  int32_t shift = 0;
  quantize_multiplier(m, mult, &shift);
  *ls = shift < 0 ? 0 : shift;
  *rs = shift < 0 ? shift : 0;
}

static void requant_params(double sx, const double *sw, int n, double so, int32_t *mult, int32_t *ls, int32_t *rs) {
  const float fx = (float)sx, fo = (float)so;
  for (int i = 0; i < n; ++i) {
    volatile float prod = fx * (float)sw[i];  // float product first, as QuantArg.scale_ is float
    round_param((double)prod / (double)fo, &mult[i], &ls[i], &rs[i]);
  }
}

static int32_t quantize_to_int8_unclamped(float real, float scale, int32_t zp) {
  volatile float t = real / scale;
  volatile float u = t + (float)zp;
  const double r = round((double)u);
  return (r >= -2147483648.0 && r <= 2147483647.0) ? (int32_t)r : INT32_MIN;
}

static void activation_range(int act, int32_t zp, float scale, int32_t *mn, int32_t *mx) {
  int32_t lo = INT8_MIN, hi = INT8_MAX;
  const int32_t q0 = quantize_to_int8_unclamped(0.0f, scale, zp), q6 = quantize_to_int8_unclamped(6.0f, scale, zp);
  if (act == MI_ACT_RELU) {
    lo = std::max(lo, q0);
  } else if (act == MI_ACT_RELU6) {
    lo = std::max(lo, q0);
    hi = std::min(hi, q6);
  }
  *mn = lo;
  *mx = hi;
}

// ---- device memory helpers ------------------------------------------------------------------------------------------
// A buffer that only grows.  Growing happens inside a run (a new shape, a longer im2col workspace), possibly with
// kernels still in flight that use the old memory, so the old allocation is neither freed there -- hipFree waits for
// the whole device -- nor reused: it is kept until the handle goes away, and the size at least doubles, which bounds
// what is kept to the final size once more.
// Test aid (mi_debug_fail_alloc): while set, every DevBuf allocation of exactly this many bytes fails.
static size_t g_fail_alloc_bytes = 0;
static hipError_t device_alloc(void **q, size_t sz) {
  if (g_fail_alloc_bytes != 0 && sz == g_fail_alloc_bytes) {
    *q = nullptr;
    return hipErrorOutOfMemory;
  }
  return hipMalloc(q, sz);
}

struct DevBuf {
  void *p = nullptr;
  size_t bytes = 0;
  std::vector<void *> retired;
  DevBuf() = default;
  DevBuf(const DevBuf &) = delete;
  DevBuf &operator=(const DevBuf &) = delete;
  ~DevBuf() { release(); }
  int ensure(size_t want) {
    if (want <= bytes) return MI_OK;
    size_t sz = p != nullptr && want < 2 * bytes ? 2 * bytes : want;
    sz = (sz + 4095) & ~(size_t)4095;
    void *q = nullptr;
    if (device_alloc(&q, sz) != hipSuccess) {
      (void)hipGetLastError();
      sz = (want + 4095) & ~(size_t)4095;  // the doubled size did not fit: exactly what is needed
      if (device_alloc(&q, sz) != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipMalloc(%zu) failed", sz);
        return MI_MEMORY_FAILED;
      }
    }
    if (p != nullptr) retired.push_back(p);
    p = q;
    bytes = sz;
    return MI_OK;
  }
  void release() {
    if (p != nullptr) (void)hipFree(p);
    for (void *q : retired) (void)hipFree(q);
    retired.clear();
    p = nullptr;
    bytes = 0;
  }
};

// Where a run takes temporary device memory from: a buffer of the handle that grows on demand, or a fixed region
// that is never reallocated.
struct Workspace {
  DevBuf *grow = nullptr;  // growable buffer, or
  void *fixed = nullptr;   // fixed region of `capacity` bytes
  size_t capacity = 0;
  static Workspace growable(DevBuf *b) {
    Workspace w;
    w.grow = b;
    return w;
  }
  static Workspace region(void *p, size_t bytes) {
    Workspace w;
    w.fixed = p;
    w.capacity = bytes;
    return w;
  }
  int get(size_t want, void **out) const {
    if (grow != nullptr) {
      int rc = grow->ensure(want);
      *out = grow->p;
      return rc;
    }
    if (want > capacity) {
      set_error("this call needs %zu bytes of scratch memory, %zu are available", want, capacity);
      return MI_PARAM_INVALID;
    }
    *out = fixed;
    return MI_OK;
  }
};

template <typename T>
static int upload(DevBuf *b, const std::vector<T> &v) {
  int rc = b->ensure(v.size() * sizeof(T) + 16);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(b->p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return MI_OK;
}

// ---- shared "requantising GEMM operand" state: packed weights + per-channel epilogue arrays ------------------------
struct RequantState {
  int n = 0, k = 0, n_pad = 0, k_pad = 0, ldw = 0;
  DevBuf w, mult, bias2, rshift, lshift, zw;
  DevBuf mult2, c2lo, c2hi, pre;  // the GEMM epilogue's per-channel constants (RequantParams::fast2)
  DevBuf w_blocked;  // the same weights in 1 KiB matrix-core blocks (2..64 activation rows, some shapes ..128); built in create or absent
  std::vector<int32_t> h_mult, h_ls, h_rs, h_bias2;
  int32_t amin = -128, amax = 127, zo = 0;
  bool has_zw = false, fast = false, fast2 = false;

  RequantParams params() const {
    RequantParams rq{};
    rq.mult = static_cast<const int32_t *>(mult.p);
    rq.bias2 = static_cast<const int32_t *>(bias2.p);
    rq.rshift = static_cast<const int32_t *>(rshift.p);
    rq.lshift = static_cast<const int32_t *>(lshift.p);
    rq.zw = static_cast<const int32_t *>(zw.p);
    rq.zo = zo;
    rq.amin = amin;
    rq.amax = amax;
    rq.has_zw = has_zw ? 1 : 0;
    rq.fast = fast ? 1 : 0;
    rq.mult2 = static_cast<const uint32_t *>(mult2.p);
    rq.c2lo = static_cast<const uint32_t *>(c2lo.p);
    rq.c2hi = static_cast<const uint32_t *>(c2hi.p);
    rq.pre = static_cast<const int32_t *>(pre.p);
    rq.fast2 = fast2 ? 1 : 0;
    return rq;
  }

  // w_nk: [n][k] row-major (already transposed if needed)
  int build(const int8_t *w_nk, int n_, int k_, const int32_t *bias, double sx, int32_t zx, double so, int32_t zo_,
            int nfilt, const double *sw, const int32_t *zws, int act, bool pack_weights, bool pack_decode = false) {
    n = n_;
    k = k_;
    n_pad = round_up(n, kNPad);
    k_pad = round_up(k, kKPad);
    ldw = weight_row_stride(k_pad);
    zo = zo_;
    const bool peroc = nfilt > 1;
    h_mult.assign(n_pad, 0);
    h_ls.assign(n_pad, 0);
    h_rs.assign(n_pad, 0);
    h_bias2.assign(n_pad, 0);
    std::vector<int32_t> m1(nfilt), l1(nfilt), r1(nfilt);
    requant_params(sx, sw, nfilt, so, m1.data(), l1.data(), r1.data());
    activation_range(act, zo, (float)so, &amin, &amax);
    std::vector<int32_t> e(n_pad, 0), zwv(n_pad, 0);
    has_zw = false;
    fast = true;
    for (int c = 0; c < n; ++c) {
      const int qi = peroc ? c : 0;
      h_mult[c] = m1[qi];
      h_ls[c] = l1[qi];
      h_rs[c] = r1[qi];
      e[c] = std::min(31, -r1[qi]);
      zwv[c] = zws[qi];
      if (zwv[c] != 0) has_zw = true;
      int32_t wsum = 0;
      const int8_t *row = w_nk + (size_t)c * k;
      for (int i = 0; i < k; ++i) wsum += row[i];
      uint32_t v = (uint32_t)k * (uint32_t)zx * (uint32_t)zwv[c] - (uint32_t)zx * (uint32_t)wsum;
      if (bias != nullptr) v += (uint32_t)bias[c];
      h_bias2[c] = (int32_t)v;
      // can the cheap rounding form be used?  needs ls == 0, 1 <= e <= 30, no saturation case, and
      // |srdhm| + 2^(e-1) representable
      const int64_t vmax = std::min<int64_t>((int64_t)1 << 31, (int64_t)k * 16384 + llabs((long long)h_bias2[c]) +
                                                                   (int64_t)k * 128 * llabs((long long)zwv[c]));
      const int64_t xmax = ((vmax * llabs((long long)h_mult[c])) >> 31) + 1;
      if (h_ls[c] != 0 || e[c] < 1 || e[c] > 30 || h_mult[c] == INT32_MIN || vmax >= ((int64_t)1 << 31) ||
          xmax + ((int64_t)1 << (e[c] - 1)) + (llabs((long long)zo) << e[c]) > INT32_MAX)
        fast = false;
    }
    for (int c = n; c < n_pad; ++c) e[c] = 1;
    if (amin > amax) fast = false;
    // constants of the GEMM's single-multiply rounding form (RequantParams::fast2).  Only that form reads the
    // accumulator register with kAccBias still in it, so the room for kAccBias is its condition alone (the first test
    // in the loop below: sum and row-sum term together stay within +-kAccBias, hence the register within [0, 2^31)).
    fast2 = fast;
    std::vector<uint32_t> m2(n_pad, 0), lo(n_pad, 0), hi(n_pad, 0);
    std::vector<int32_t> prev(n_pad, 0);
    for (int c = 0; c < n && fast2; ++c) {
      if (h_mult[c] < 0 || (int64_t)k * 16384 + (int64_t)k * 128 * llabs((long long)zwv[c]) > (int64_t)kAccBias) {
        fast2 = false;
        break;
      }
      m2[c] = (uint32_t)h_mult[c] << 1;
      const uint64_t c2 = (uint64_t)(2 * ((int64_t)h_bias2[c] - (int64_t)kAccBias)) * (uint64_t)(int64_t)h_mult[c] +
                          ((uint64_t)1 << 31);
      if ((int64_t)c2 >= 0) {  // the epilogue reads the sign of x off the carry of a * mult2 + c2
        fast2 = false;
        break;
      }
      lo[c] = (uint32_t)c2;
      hi[c] = (uint32_t)(c2 >> 32);
      prev[c] = (int32_t)(((uint32_t)1 << e[c]) >> 1) + (int32_t)((uint32_t)zo << e[c]) - 1;
    }
    int rc;
    if ((rc = upload(&mult2, m2)) != MI_OK) return rc;
    if ((rc = upload(&c2lo, lo)) != MI_OK) return rc;
    if ((rc = upload(&c2hi, hi)) != MI_OK) return rc;
    if ((rc = upload(&pre, prev)) != MI_OK) return rc;
    if ((rc = upload(&mult, h_mult)) != MI_OK) return rc;
    if ((rc = upload(&bias2, h_bias2)) != MI_OK) return rc;
    if ((rc = upload(&rshift, e)) != MI_OK) return rc;
    if ((rc = upload(&lshift, h_ls)) != MI_OK) return rc;
    if ((rc = upload(&zw, zwv)) != MI_OK) return rc;
    if (pack_weights) {
      std::vector<int8_t> packed((size_t)n_pad * ldw, 0);
      for (int c = 0; c < n; ++c) memcpy(packed.data() + (size_t)c * ldw, w_nk + (size_t)c * k, (size_t)k);
      if ((rc = upload(&w, packed)) != MI_OK) return rc;
      if (pack_decode) {
        // The blocked copy is an optimisation for 2..64 activation rows (some shapes: ..128), not a requirement: without it those row
        // counts run on the v_dot4 kernel (two rows) or the GEMM tiles.  A device that has no room for it still gets
        // a working handle.
        rc = w_blocked.ensure((size_t)n_pad * k_pad);
        if (rc == MI_OK)
          rc = launch_block_weights(static_cast<const int8_t *>(w.p), n_pad, k_pad, ldw,
                                    static_cast<int8_t *>(w_blocked.p), nullptr);
        if (rc == MI_OK && hipStreamSynchronize(nullptr) != hipSuccess) rc = MI_ERROR;  // runs may come in on any stream
        if (rc != MI_OK) {
          (void)hipGetLastError();
          w_blocked.release();
          set_error("");
        }
      }
    }
    return MI_OK;
  }

  void release() {
    w.release();
    w_blocked.release();
    mult.release();
    bias2.release();
    rshift.release();
    lshift.release();
    zw.release();
    mult2.release();
    c2lo.release();
    c2hi.release();
    pre.release();
  }
};

static int check_filter_quant(int nfilt, int channels, const double *scales, const int32_t *zps) {
  if (scales == nullptr || zps == nullptr) {
    set_error("filter quant params are null");
    return MI_NULL_PTR;
  }
  if (nfilt != 1 && nfilt != channels) {
    set_error("filter_quant_num must be 1 or the channel count (%d), got %d", channels, nfilt);
    return MI_PARAM_INVALID;
  }
  return MI_OK;
}

static std::vector<int8_t> to_nk(const int8_t *w, int n, int k, int b_transpose) {
  std::vector<int8_t> out((size_t)n * k);
  if (b_transpose) {
    memcpy(out.data(), w, out.size());
  } else {
    constexpr int kTile = 64;  // both the reads and the writes of a tile stay within a few cache lines
    for (int k0 = 0; k0 < k; k0 += kTile)
      for (int c0 = 0; c0 < n; c0 += kTile)
        for (int kk = k0; kk < std::min(k, k0 + kTile); ++kk)
          for (int c = c0; c < std::min(n, c0 + kTile); ++c) out[(size_t)c * k + kk] = w[(size_t)kk * n + c];
  }
  return out;
}

// The weight layout that a model converted for the ARM dot-product kernel carries (RowMajor2Row4x16MajorInt8 for
// transpose_b, RowMajor2Col4x16MajorInt8 otherwise, nnacl/int8/matmul_int8.c:143-156,770-784; both give the same
// bytes): blocks [n / 16][k / 4] of 16 channels x 4 K-bytes, channel-major inside a block, with the channel count
// padded to 16 and K to 4.  Returns [n][k] row-major (the inverse that MatmulDynamicSdotInt8Unpack computes,
// mindspore/lite/src/litert/runtime_packed_node_pass.cc:158-192).
static std::vector<int8_t> unpack_4x16(const int8_t *packed, int n, int k) {
  const size_t k4 = (size_t)round_up(k, 4);
  std::vector<int8_t> out((size_t)n * k);
  for (int c = 0; c < n; ++c) {
    const int8_t *blk = packed + (size_t)(c / 16) * k4 * 16 + (size_t)(c % 16) * 4;
    int8_t *row = out.data() + (size_t)c * k;
    for (int i = 0; i < k; ++i) row[i] = blk[(size_t)(i / 4) * 64 + (i % 4)];
  }
  return out;
}

// Activations must reach the GEMM/GEMV kernels as 16-byte aligned rows of k16 bytes; returns the pointer/stride to
// use, copying through `ws` when the caller's layout does not qualify.
static int prepare_rows(const int8_t *a, int rows, int k, const Workspace &ws, hipStream_t stream,
                        const int8_t **a_out, int64_t *lda_out, int *k16_out) {
  const int k16 = round_up(k, 16);
  if (k16 == k && (reinterpret_cast<uintptr_t>(a) & 15) == 0) {
    *a_out = a;
    *lda_out = k;
    *k16_out = k;
    return MI_OK;
  }
  void *buf = nullptr;
  int rc = ws.get((size_t)rows * k16, &buf);
  if (rc != MI_OK) return rc;
  rc = launch_pad_rows(a, k, rows, k, static_cast<int8_t *>(buf), k16, stream);
  if (rc != MI_OK) return rc;
  *a_out = static_cast<const int8_t *>(buf);
  *lda_out = k16;
  *k16_out = k16;
  return MI_OK;
}

// The GEMM kernels write rows with vector stores; when the caller's row length or base address does not allow that,
// they write to a padded scratch output which is then compacted into the caller's tensor.
static int run_requant_gemm(RequantState &st, const int8_t *a, int64_t lda, int rows, int k16, int8_t *c,
                            const Workspace &c_ws, hipStream_t stream) {
  const RequantParams rq = st.params();
  WeightView w{static_cast<const int8_t *>(st.w.p), st.k_pad, st.ldw, nullptr};
  // one row: the dot kernel on the row-major weights; 2..64 rows (..128 against at most 4096 channels and K >= 1024): the matrix-core decode kernel on the blocked copy
  // made at create time -- a handle without it runs two rows on the dot kernel and 3..64 on the GEMM tiles
  const bool skinny = rows <= kGemvDotRows ? (int64_t)rows * k16 <= 150 * 1024
                                           : gemv_takes_rows(rows, st.n, st.k_pad) && st.w_blocked.p != nullptr && st.k_pad <= 1 << 20;
  if (skinny) {
    if (rows >= 2) w.blocked = static_cast<const int8_t *>(st.w_blocked.p);  // (may be absent: two rows then take the v_dot4 kernel)
    return launch_gemv_requant(a, lda, rows, k16, w, st.n, rq, c, st.n, stream);
  }
  if ((st.n & 3) == 0 && (reinterpret_cast<uintptr_t>(c) & 3) == 0)
    return launch_gemm_requant(a, lda, rows, k16, w, st.n, rq, c, st.n, stream);
  const int n4 = round_up(st.n, 4);
  void *buf = nullptr;
  int rc = c_ws.get((size_t)rows * n4, &buf);
  if (rc != MI_OK) return rc;
  rc = launch_gemm_requant(a, lda, rows, k16, w, n4, rq, static_cast<int8_t *>(buf), n4, stream);
  if (rc != MI_OK) return rc;
  return launch_copy_rows(buf, n4, rows, st.n, c, st.n, stream);
}

}  // namespace mi

using namespace mi;

// =====================================================================================================================
struct mi_matmul {
  RequantState st;  // weight matrix 0
  std::vector<std::unique_ptr<RequantState>> more;  // weight matrices 1 .. b_batch - 1 of a batched constant weight
  DevBuf a_ws, c_ws, h_in, h_out;
  int b_batch() const { return 1 + (int)more.size(); }
  RequantState &state(int b) { return b == 0 ? st : *more[(size_t)b - 1]; }
};

struct mi_conv {
  mi_conv_desc d;
  bool depthwise = false, direct_1x1 = false, dw_fast = false;
  int fill = 0;
  RequantState st;
  DevBuf w16, dw_bias, dw_bias_folded, col_ws, c_ws, h_in, h_out;
  DevBuf fill16;  // 16 bytes of `fill`: where the gathering GEMM loader reads taps outside the image
};

struct mi_dynquant {
  int symmetric = 0;
  DevBuf partials, params, h_in, h_out, h_params;
};

struct mi_dynmm {
  int n = 0, k = 0, n_pad = 0, k_pad = 0, ldw = 0, act = 0;
  int32_t zw0 = 0;
  bool has_bias = false;
  DevBuf w, wscale, wsum, bias, a_ws, c_ws, h_in, h_out, h_params;
  DevBuf w_blocked;  // the weights in 1 KiB matrix-core blocks for 2..64 activation rows (some shapes ..128); built in create or absent
};

// No C++ exception may cross the C ABI: host allocations in the create calls can throw.
template <typename F>
static int guarded(const char *what, F &&f) {
  try {
    return f();
  } catch (const std::bad_alloc &) {
    set_error("%s: out of host memory", what);
    return MI_MEMORY_FAILED;
  } catch (...) {
    set_error("%s: unexpected exception", what);
    return MI_ERROR;
  }
}

extern "C" {

int mi_init(int device) {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    set_error("no HIP device visible");
    return MI_NOT_SUPPORT;
  }
  if (device < 0 || device >= count) {
    set_error("device %d out of range (%d visible)", device, count);
    return MI_PARAM_INVALID;
  }
  hipDeviceProp_t prop;
  MI_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error("device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
    return MI_NOT_SUPPORT;
  }
  MI_HIP_CHECK(hipSetDevice(device));
  int rc = gemv_prepare_device();
  if (rc != MI_OK) return rc;
  if (device < kMaxDevices && g_scratch_ptr[device] == nullptr) {
    void *ptr = nullptr;
    MI_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));  // this device's copy of the array
    g_scratch_ptr[device] = ptr;
  }
  g_device = device;
  return MI_OK;
}

int mi_device_malloc(size_t bytes, void **out_dev) {
  if (out_dev == nullptr) return MI_NULL_PTR;
  *out_dev = nullptr;
  if (bytes == 0) {
    set_error("mi_device_malloc: zero bytes");
    return MI_PARAM_INVALID;
  }
  if (ensure_device() != MI_OK) return MI_ERROR;
  const size_t sz = (bytes + 255) & ~(size_t)255;
  if (hipMalloc(out_dev, sz) != hipSuccess) {
    *out_dev = nullptr;
    set_error("hipMalloc(%zu) failed", sz);
    return MI_MEMORY_FAILED;
  }
  return MI_OK;
}

int mi_device_free(void *dev) {
  if (dev == nullptr) return MI_OK;
  if (ensure_device() != MI_OK) return MI_ERROR;
  MI_HIP_CHECK(hipFree(dev));
  return MI_OK;
}

int mi_host_malloc(size_t bytes, void **out_host) {
  if (out_host == nullptr) return MI_NULL_PTR;
  *out_host = nullptr;
  if (bytes == 0) {
    set_error("mi_host_malloc: zero bytes");
    return MI_PARAM_INVALID;
  }
  if (ensure_device() != MI_OK) return MI_ERROR;
  if (hipHostMalloc(out_host, bytes, hipHostMallocDefault) != hipSuccess) {
    *out_host = nullptr;
    set_error("hipHostMalloc(%zu) failed", bytes);
    return MI_MEMORY_FAILED;
  }
  return MI_OK;
}

int mi_host_free(void *host) {
  if (host == nullptr) return MI_OK;
  if (ensure_device() != MI_OK) return MI_ERROR;
  MI_HIP_CHECK(hipHostFree(host));
  return MI_OK;
}

int mi_copy_to_device(void *dst_dev, const void *src_host, size_t bytes, void *stream) {
  if (bytes == 0) return MI_OK;
  if (dst_dev == nullptr || src_host == nullptr) return MI_NULL_PTR;
  if (ensure_device() != MI_OK) return MI_ERROR;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI_HIP_CHECK(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, s));
  MI_HIP_CHECK(counted_sync(s));  // the caller may reuse src_host at once (the runtime recycles tensor memory)
  return MI_OK;
}

int mi_copy_to_host(void *dst_host, const void *src_dev, size_t bytes, void *stream) {
  if (bytes == 0) return MI_OK;
  if (dst_host == nullptr || src_dev == nullptr) return MI_NULL_PTR;
  if (ensure_device() != MI_OK) return MI_ERROR;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI_HIP_CHECK(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, s));
  MI_HIP_CHECK(counted_sync(s));
  return MI_OK;
}

int mi_copy_to_host_async(void *dst_host, const void *src_dev, size_t bytes, void *stream) {
  if (bytes == 0) return MI_OK;
  if (dst_host == nullptr || src_dev == nullptr) return MI_NULL_PTR;
  if (ensure_device() != MI_OK) return MI_ERROR;
  MI_HIP_CHECK(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
  return MI_OK;
}

int64_t mi_debug_sync_count(void) { return g_sync_count.load(std::memory_order_relaxed); }

int mi_stream_create(void **out_stream) {
  if (out_stream == nullptr) return MI_NULL_PTR;
  *out_stream = nullptr;
  if (ensure_device() != MI_OK) return MI_ERROR;
  hipStream_t s = nullptr;
  MI_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));  // default priority; independent of the null stream
  *out_stream = s;
  return MI_OK;
}

int mi_stream_destroy(void *stream) {
  if (stream == nullptr) return MI_OK;
  if (ensure_device() != MI_OK) return MI_ERROR;
  MI_HIP_CHECK(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return MI_OK;
}

int mi_stream_synchronize(void *stream) {
  if (ensure_device() != MI_OK) return MI_ERROR;
  MI_HIP_CHECK(counted_sync(static_cast<hipStream_t>(stream)));
  return MI_OK;
}

int mi_debug_fail_alloc(size_t bytes) {
  g_fail_alloc_bytes = bytes == 0 ? 0 : (bytes + 4095) & ~(size_t)4095;
  return MI_OK;
}

const char *mi_last_error(void) { return g_err; }
const char *mi_version(void) { return "mi355x_int8 0.1 (gfx950)"; }

int mi_quantize_multiplier(double real_multiplier, int32_t *multiplier, int32_t *left_shift, int32_t *right_shift) {
  if (multiplier == nullptr || left_shift == nullptr || right_shift == nullptr) return MI_NULL_PTR;
  round_param(real_multiplier, multiplier, left_shift, right_shift);
  return MI_OK;
}

int mi_quantize_multiplier_single(double real_multiplier, int32_t *multiplier, int32_t *left_shift,
                                  int32_t *right_shift) {
  if (multiplier == nullptr || left_shift == nullptr || right_shift == nullptr) return MI_NULL_PTR;
  if (!(real_multiplier >= 0.0 && real_multiplier < 4294967296.0)) {
    set_error("mi_quantize_multiplier_single: the multiplier must be in [0, 2^32)");
    return MI_PARAM_INVALID;
  }
  // the reference converts the double's VALUE to uint32 here, so every multiplier below 1 gives
  // (0x40000000, 0, -126); reproduced as it is
  const uint32_t bits = (uint32_t)real_multiplier;
  *multiplier = (int32_t)(((bits & 0x007FFFFFu) | 0x00800000u) << 7);
  const int32_t shift = -(127 + 31 - 32 - (int32_t)(bits >> 23));
  *left_shift = shift < 0 ? 0 : shift;
  *right_shift = shift < 0 ? shift : 0;
  return MI_OK;
}

int mi_activation_range(int32_t act_type, int32_t out_zp, double out_scale, int32_t *act_min, int32_t *act_max) {
  if (act_min == nullptr || act_max == nullptr) return MI_NULL_PTR;
  activation_range(act_type, out_zp, (float)out_scale, act_min, act_max);
  return MI_OK;
}

int mi_requant_params(double in_scale, const double *filter_scales, int32_t n, double out_scale, int32_t *multiplier,
                      int32_t *left_shift, int32_t *right_shift) {
  if (filter_scales == nullptr || multiplier == nullptr || left_shift == nullptr || right_shift == nullptr)
    return MI_NULL_PTR;
  if (n < 0) return MI_PARAM_INVALID;
  requant_params(in_scale, filter_scales, n, out_scale, multiplier, left_shift, right_shift);
  return MI_OK;
}

int32_t mi_multiply_by_quantized_multiplier(int32_t value, int32_t multiplier, int32_t left_shift,
                                            int32_t right_shift) {
  return mul_by_quant_mult(value, multiplier, left_shift, right_shift);
}

// ---------------------------------------------------------------------------------------------------------- matmul
static int mi_matmul_create_impl(const mi_matmul_desc *d, const int8_t *weight_host, const int32_t *bias_host, mi_matmul **out) {
  if (d == nullptr || weight_host == nullptr || out == nullptr) {
    set_error("mi_matmul_create: null argument");
    return MI_NULL_PTR;
  }
  *out = nullptr;
  if (d->deep <= 0 || d->col <= 0 || (d->act_type != MI_ACT_NONE && d->act_type != MI_ACT_RELU &&
                                      d->act_type != MI_ACT_RELU6)) {
    set_error("mi_matmul_create: bad shape/activation deep=%d col=%d act=%d", d->deep, d->col, d->act_type);
    return MI_PARAM_INVALID;
  }
  if ((d->flags & ~MI_MATMUL_NO_DECODE_PACK) != 0) {
    set_error("mi_matmul_create: unknown flags 0x%x", d->flags);
    return MI_PARAM_INVALID;
  }
  int rc = check_filter_quant(d->filter_quant_num, d->col, d->filter_scales, d->filter_zps);
  if (rc != MI_OK) return rc;
  if ((rc = ensure_device()) != MI_OK) return rc;
  std::unique_ptr<mi_matmul> owner(new (std::nothrow) mi_matmul());  // the buffers free themselves if anything below throws
  mi_matmul *h = owner.get();
  if (h == nullptr) return MI_MEMORY_FAILED;
  if (d->b_batch < 0 || d->b_batch > (1 << 16)) {
    set_error("mi_matmul_create: b_batch=%d", d->b_batch);
    return MI_PARAM_INVALID;
  }
  // every matrix of a batched weight gets its own packed copy and folded bias; quant parameters and bias are shared
  // (TransferB, LK/int8/matmul_base_int8.cc:360-384)
  const int b_batch = d->b_batch > 1 ? d->b_batch : 1;
  for (int b = 0; b < b_batch; ++b) {
    if (b > 0) {
      h->more.emplace_back(new (std::nothrow) RequantState());
      if (h->more.back() == nullptr) return MI_MEMORY_FAILED;
    }
    const std::vector<int8_t> w_nk = to_nk(weight_host + (size_t)b * d->col * d->deep, d->col, d->deep, d->b_transpose);
    rc = h->state(b).build(w_nk.data(), d->col, d->deep, bias_host, d->in_scale, d->in_zp, d->out_scale, d->out_zp,
                           d->filter_quant_num, d->filter_scales, d->filter_zps, d->act_type, true,
                           (d->flags & MI_MATMUL_NO_DECODE_PACK) == 0);
    if (rc != MI_OK) return rc;
  }
  *out = owner.release();
  return MI_OK;
}

int mi_matmul_create(const mi_matmul_desc *d, const int8_t *weight_host, const int32_t *bias_host, mi_matmul **out) {
  return guarded("mi_matmul_create", [&] { return mi_matmul_create_impl(d, weight_host, bias_host, out); });
}

int mi_matmul_reserve(mi_matmul *h, int32_t max_rows) {
  if (h == nullptr) return MI_NULL_PTR;
  if (max_rows < 0) return MI_PARAM_INVALID;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  // sized for the worst case of either workspace: whether a run needs them also depends on its pointers
  if ((rc = h->a_ws.ensure((size_t)max_rows * round_up(h->st.k, 16))) != MI_OK) return rc;
  return h->c_ws.ensure((size_t)max_rows * round_up(h->st.n, 4));
}

int mi_matmul_run(mi_matmul *h, const int8_t *a_dev, int32_t rows, int8_t *c_dev, void *stream) {
  if (h == nullptr || a_dev == nullptr || c_dev == nullptr) {
    set_error("mi_matmul_run: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) {
    set_error("mi_matmul_run: rows=%d", rows);
    return MI_PARAM_INVALID;
  }
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  if ((rc = prepare_rows(a_dev, rows, h->st.k, Workspace::growable(&h->a_ws), s, &a, &lda, &k16)) != MI_OK) return rc;
  return run_requant_gemm(h->st, a, lda, rows, k16, c_dev, Workspace::growable(&h->c_ws), s);
}

int mi_matmul_run_batched(mi_matmul *h, const int8_t *a_dev, int32_t rows, int32_t batch, const int32_t *a_offsets,
                          const int32_t *b_offsets, int8_t *c_dev, void *stream) {
  if (h == nullptr || a_dev == nullptr || c_dev == nullptr || a_offsets == nullptr || b_offsets == nullptr) {
    set_error("mi_matmul_run_batched: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0 || batch < 0) {
    set_error("mi_matmul_run_batched: rows=%d batch=%d", rows, batch);
    return MI_PARAM_INVALID;
  }
  for (int i = 0; i < batch; ++i) {
    if (a_offsets[i] < 0 || b_offsets[i] < 0 || b_offsets[i] >= h->b_batch()) {
      set_error("mi_matmul_run_batched: output matrix %d takes activation matrix %d and weight matrix %d of %d", i,
                a_offsets[i], b_offsets[i], h->b_batch());
      return MI_PARAM_INVALID;
    }
  }
  if (rows == 0 || batch == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t a_mat = (size_t)rows * h->st.k, c_mat = (size_t)rows * h->st.n;
  // one launch per output matrix, in order on the stream (so the shared workspaces are reused safely), as the
  // reference runs one ParallelLaunch per batch (LK/int8/matmul_base_int8.cc:549-568)
  for (int i = 0; i < batch; ++i) {
    const int8_t *a = nullptr;
    int64_t lda = 0;
    int k16 = 0;
    if ((rc = prepare_rows(a_dev + (size_t)a_offsets[i] * a_mat, rows, h->st.k, Workspace::growable(&h->a_ws), s, &a, &lda,
                           &k16)) != MI_OK)
      return rc;
    if ((rc = run_requant_gemm(h->state(b_offsets[i]), a, lda, rows, k16, c_dev + (size_t)i * c_mat,
                               Workspace::growable(&h->c_ws), s)) != MI_OK)
      return rc;
  }
  return MI_OK;
}

int mi_matmul_run_group(mi_matmul *const *handles, int32_t count, const int8_t *a_dev, int32_t rows,
                        int8_t *const *c_dev, void *stream) {
  if (handles == nullptr || a_dev == nullptr || c_dev == nullptr) {
    set_error("mi_matmul_run_group: null argument");
    return MI_NULL_PTR;
  }
  if (count < 1 || rows < 0) {
    set_error("mi_matmul_run_group: count=%d rows=%d", count, rows);
    return MI_PARAM_INVALID;
  }
  for (int i = 0; i < count; ++i) {
    if (handles[i] == nullptr || c_dev[i] == nullptr) {
      set_error("mi_matmul_run_group: member %d is null", i);
      return MI_NULL_PTR;
    }
    if (handles[i]->st.k != handles[0]->st.k) {
      set_error("mi_matmul_run_group: member %d has deep %d, member 0 has %d", i, handles[i]->st.k, handles[0]->st.k);
      return MI_PARAM_INVALID;
    }
  }
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  // the activation rows are brought into the kernels' form once, for all members
  if ((rc = prepare_rows(a_dev, rows, handles[0]->st.k, Workspace::growable(&handles[0]->a_ws), s, &a, &lda, &k16)) != MI_OK)
    return rc;
  // decode-sized runs of up to four members go out as one launch; anything else runs member by member
  bool one_launch = count >= 2 && count <= 4 && rows <= kGemvGroupMaxRows;
  for (int i = 0; i < count && one_launch; ++i)
    one_launch = rows <= kGemvDotRows ? (int64_t)rows * k16 <= 150 * 1024
                                      : handles[i]->st.w_blocked.p != nullptr && handles[i]->st.k_pad <= 1 << 20;
  if (one_launch) {
    WeightView wv[4];
    RequantParams rq[4];
    int n[4];
    for (int i = 0; i < count; ++i) {
      const RequantState &st = handles[i]->st;
      wv[i] = WeightView{static_cast<const int8_t *>(st.w.p), st.k_pad, st.ldw, static_cast<const int8_t *>(st.w_blocked.p)};
      rq[i] = st.params();
      n[i] = st.n;
    }
    return launch_gemv_group(a, lda, rows, k16, count, wv, n, rq, c_dev, s);
  }
  for (int i = 0; i < count; ++i)
    if ((rc = run_requant_gemm(handles[i]->st, a, lda, rows, k16, c_dev[i], Workspace::growable(&handles[i]->c_ws), s)) != MI_OK)
      return rc;
  return MI_OK;
}

int mi_matmul_run_noalloc(mi_matmul *h, const int8_t *a_dev, int32_t rows, int8_t *c_dev, void *stream) {
  if (h == nullptr || a_dev == nullptr || c_dev == nullptr) {
    set_error("mi_matmul_run_noalloc: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) {
    set_error("mi_matmul_run_noalloc: rows=%d", rows);
    return MI_PARAM_INVALID;
  }
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  void *base = g_device < kMaxDevices ? g_scratch_ptr[g_device] : nullptr;
  if (base == nullptr) {
    set_error("mi_matmul_run_noalloc: no scratch memory on device %d", g_device);
    return MI_ERROR;
  }
  // the padded activation rows first, the padded output behind them; a part is only needed when the operand's shape
  // or this call's pointer alignment asks for it, and only the needed parts count against the maximum (so a shape
  // that passes with aligned pointers can be refused with misaligned ones)
  const size_t a_bytes = round_up64((int64_t)rows * round_up(h->st.k, 16), 256);
  const size_t c_bytes = (size_t)rows * round_up(h->st.n, 4);
  const bool a_padded = (h->st.k & 15) != 0, c_padded = (h->st.n & 3) != 0;
  const bool a_unaligned = (reinterpret_cast<uintptr_t>(a_dev) & 15) != 0;
  const bool c_unaligned = (reinterpret_cast<uintptr_t>(c_dev) & 3) != 0;
  const size_t need = ((a_padded || a_unaligned) ? a_bytes : 0) + ((c_padded || c_unaligned) ? c_bytes : 0);
  if (need > kScratchBytes) {
    set_error("mi_matmul_run_noalloc: %d rows of this MatMul (deep %d, col %d) need %zu bytes of scratch memory, the "
              "maximum is %zu; use mi_matmul_run", rows, h->st.k, h->st.n, need, kScratchBytes);
    return MI_PARAM_INVALID;
  }
  unsigned char *p = static_cast<unsigned char *>(base);
  const Workspace a_ws = Workspace::region(p, a_bytes);
  const Workspace c_ws = Workspace::region(p + ((a_padded || a_unaligned) ? a_bytes : 0), c_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  if ((rc = prepare_rows(a_dev, rows, h->st.k, a_ws, s, &a, &lda, &k16)) != MI_OK) return rc;
  return run_requant_gemm(h->st, a, lda, rows, k16, c_dev, c_ws, s);
}

int mi_matmul_run_host(mi_matmul *h, const int8_t *a_host, int32_t rows, int8_t *c_host) {
  if (h == nullptr || a_host == nullptr || c_host == nullptr) {
    set_error("mi_matmul_run_host: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) return MI_PARAM_INVALID;
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  const size_t in_bytes = (size_t)rows * h->st.k, out_bytes = (size_t)rows * h->st.n;
  if ((rc = h->h_in.ensure(in_bytes)) != MI_OK || (rc = h->h_out.ensure(out_bytes)) != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(h->h_in.p, a_host, in_bytes, hipMemcpyHostToDevice));
  rc = mi_matmul_run(h, static_cast<const int8_t *>(h->h_in.p), rows, static_cast<int8_t *>(h->h_out.p), nullptr);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(c_host, h->h_out.p, out_bytes, hipMemcpyDeviceToHost));
  return MI_OK;
}

int mi_matmul_get_params(const mi_matmul *h, int32_t *multiplier, int32_t *left_shift, int32_t *right_shift,
                         int32_t *folded_bias, int32_t *act_min, int32_t *act_max) {
  if (h == nullptr) return MI_NULL_PTR;
  const size_t bytes = (size_t)h->st.n * sizeof(int32_t);
  if (multiplier) memcpy(multiplier, h->st.h_mult.data(), bytes);
  if (left_shift) memcpy(left_shift, h->st.h_ls.data(), bytes);
  if (right_shift) memcpy(right_shift, h->st.h_rs.data(), bytes);
  if (folded_bias) memcpy(folded_bias, h->st.h_bias2.data(), bytes);
  if (act_min) *act_min = h->st.amin;
  if (act_max) *act_max = h->st.amax;
  return MI_OK;
}

void mi_matmul_destroy(mi_matmul *h) { delete h; }  // every DevBuf member frees its device memory

// ------------------------------------------------------------------------------------------------------------ conv
int mi_conv_same_pad(int32_t in, int32_t kernel, int32_t stride, int32_t dilation, int32_t *pad_before,
                     int32_t *pad_after, int32_t *out) {
  if (pad_before == nullptr || pad_after == nullptr || out == nullptr) return MI_NULL_PTR;
  if (stride <= 0 || kernel <= 0 || dilation <= 0 || in <= 0) return MI_PARAM_INVALID;
  const int o = (in + stride - 1) / stride;
  const int all = (o - 1) * stride + (kernel - 1) * dilation + 1 - in;
  *out = o;
  if (all < 0) {
    *pad_before = *pad_after = 0;
  } else {
    *pad_before = all / 2;
    *pad_after = all - all / 2;
  }
  return MI_OK;
}

static int mi_conv_create_impl(const mi_conv_desc *d, const int8_t *weight_host, const int32_t *bias_host, mi_conv **out) {
  if (d == nullptr || weight_host == nullptr || out == nullptr) {
    set_error("mi_conv_create: null argument");
    return MI_NULL_PTR;
  }
  *out = nullptr;
  if (d->in_channel <= 0 || d->out_channel <= 0 || d->kernel_h <= 0 || d->kernel_w <= 0 || d->stride_h <= 0 ||
      d->stride_w <= 0 || d->dilation_h <= 0 || d->dilation_w <= 0 || d->pad_u < 0 || d->pad_d < 0 || d->pad_l < 0 ||
      d->pad_r < 0 || d->group <= 0 ||
      (d->act_type != MI_ACT_NONE && d->act_type != MI_ACT_RELU && d->act_type != MI_ACT_RELU6)) {
    set_error("mi_conv_create: bad descriptor");
    return MI_PARAM_INVALID;
  }
  const bool depthwise = d->group > 1 && d->group == d->in_channel && d->group == d->out_channel;
  if (d->group != 1 && !depthwise) {
    set_error("grouped convolution (group=%d) is left to the builtin kernel", d->group);
    return MI_NOT_SUPPORT;
  }
  if ((d->flags & ~MI_CONV_3X3_EXACT) != 0) {
    set_error("mi_conv_create: unknown flags 0x%x", d->flags);
    return MI_PARAM_INVALID;
  }
  if (!depthwise && d->kernel_h == 3 && d->kernel_w == 3 && d->stride_h == 1 && d->stride_w == 1 &&
      d->dilation_h == 1 && d->dilation_w == 1 && (d->flags & MI_CONV_3X3_EXACT) == 0) {
    set_error("3x3 stride-1 dilation-1 convolution is left to the builtin (Winograd) kernel; MI_CONV_3X3_EXACT "
              "selects the exact convolution the reference runs on ARM64 cores with dot-product instructions");
    return MI_NOT_SUPPORT;
  }
  int rc = check_filter_quant(d->filter_quant_num, d->out_channel, d->filter_scales, d->filter_zps);
  if (rc != MI_OK) return rc;
  if ((rc = ensure_device()) != MI_OK) return rc;
  std::unique_ptr<mi_conv> owner(new (std::nothrow) mi_conv());  // the buffers free themselves if anything below throws
  mi_conv *h = owner.get();
  if (h == nullptr) return MI_MEMORY_FAILED;
  h->d = *d;
  h->d.filter_scales = nullptr;
  h->d.filter_zps = nullptr;
  h->depthwise = depthwise;
  const int oc = d->out_channel;
  if (depthwise) {
    const int plane = d->kernel_h * d->kernel_w;
    // requant arrays only; the folded bias is not used (zero points are applied to the operands)
    std::vector<int8_t> dummy((size_t)oc, 0);
    rc = h->st.build(dummy.data(), oc, 1, nullptr, d->in_scale, 0, d->out_scale, d->out_zp, d->filter_quant_num,
                     d->filter_scales, d->filter_zps, d->act_type, false);
    std::vector<int16_t> w16((size_t)plane * oc);
    for (int c = 0; c < oc; ++c) {
      const int32_t z = d->filter_quant_num > 1 ? d->filter_zps[c] : d->filter_zps[0];
      for (int t = 0; t < plane; ++t) w16[(size_t)t * oc + c] = (int16_t)((int32_t)weight_host[(size_t)c * plane + t] - z);
    }
    std::vector<int32_t> b(oc, 0);
    if (bias_host != nullptr) memcpy(b.data(), bias_host, (size_t)oc * sizeof(int32_t));
    // For the channel-vectorised kernel: a tap outside the image reads as the input zero point, so that
    // (x - zx) * w vanishes there, and -zx * sum_t(w) moves into the bias once: bias' = bias - zx8 * sum_t w16[t][c].
    // Identical to the reference's sum over the valid taps modulo 2^32.
    const int32_t zx8 = (int32_t)(int8_t)d->in_zp;
    std::vector<int32_t> bf(oc, 0);
    h->dw_fast = h->st.amin <= h->st.amax;
    for (int c = 0; c < oc; ++c) {
      uint32_t wsum = 0;
      for (int t = 0; t < plane; ++t) wsum += (uint32_t)(int32_t)w16[(size_t)t * oc + c];
      bf[c] = (int32_t)((uint32_t)b[c] - (uint32_t)zx8 * wsum);
      // the cheap rounding form needs: no left shift, 1 <= e <= 30, no saturating product, nothing leaves int32
      const int32_t mult = h->st.h_mult[c], e = std::min(31, -h->st.h_rs[c]);
      const int64_t vmax = (int64_t)plane * 255 * 255 + llabs((long long)b[c]);
      const int64_t xmax = ((vmax * llabs((long long)mult)) >> 31) + 1;
      if (h->st.h_ls[c] != 0 || e < 1 || e > 30 || mult == INT32_MIN || vmax >= ((int64_t)1 << 31) ||
          xmax + ((int64_t)1 << (e - 1)) + llabs((long long)d->out_zp) + 1 > INT32_MAX)
        h->dw_fast = false;
    }
    if (rc == MI_OK) rc = upload(&h->w16, w16);
    if (rc == MI_OK) rc = upload(&h->dw_bias, b);
    if (rc == MI_OK) rc = upload(&h->dw_bias_folded, bf);
  } else {
    const int kdim = d->kernel_h * d->kernel_w * d->in_channel;
    const bool is_1x1 = d->kernel_h == 1 && d->kernel_w == 1;
    const bool trivial_geom = d->stride_h == 1 && d->stride_w == 1 && d->pad_u == 0 && d->pad_d == 0 &&
                              d->pad_l == 0 && d->pad_r == 0;
    h->direct_1x1 = is_1x1 && trivial_geom;
    h->fill = is_1x1 ? 0 : d->in_zp;
    rc = h->st.build(weight_host, oc, kdim, bias_host, d->in_scale, d->in_zp, d->out_scale, d->out_zp,
                     d->filter_quant_num, d->filter_scales, d->filter_zps, d->act_type, true);
    if (rc == MI_OK) rc = upload(&h->fill16, std::vector<int8_t>(16, (int8_t)h->fill));
  }
  if (rc != MI_OK) {
    return rc;
  }
  *out = owner.release();
  return MI_OK;
}

int mi_conv_create(const mi_conv_desc *d, const int8_t *weight_host, const int32_t *bias_host, mi_conv **out) {
  return guarded("mi_conv_create", [&] { return mi_conv_create_impl(d, weight_host, bias_host, out); });
}

int mi_conv_out_shape(const mi_conv *h, int32_t in_h, int32_t in_w, int32_t *out_h, int32_t *out_w) {
  if (h == nullptr || out_h == nullptr || out_w == nullptr) return MI_NULL_PTR;
  const mi_conv_desc &d = h->d;
  const int eh = (d.kernel_h - 1) * d.dilation_h + 1, ew = (d.kernel_w - 1) * d.dilation_w + 1;
  if (in_h <= 0 || in_w <= 0 || in_h + d.pad_u + d.pad_d < eh || in_w + d.pad_l + d.pad_r < ew) {
    set_error("mi_conv_out_shape: input %dx%d too small", in_h, in_w);
    return MI_PARAM_INVALID;
  }
  *out_h = (in_h + d.pad_u + d.pad_d - eh) / d.stride_h + 1;
  *out_w = (in_w + d.pad_l + d.pad_r - ew) / d.stride_w + 1;
  return MI_OK;
}

int mi_conv_reserve(mi_conv *h, int32_t batch, int32_t in_h, int32_t in_w) {
  if (h == nullptr) return MI_NULL_PTR;
  if (batch < 0) return MI_PARAM_INVALID;
  int oh = 0, ow = 0;
  int rc = mi_conv_out_shape(h, in_h, in_w, &oh, &ow);
  if (rc != MI_OK) return rc;
  if (h->depthwise || batch == 0) return MI_OK;
  if ((rc = ensure_device()) != MI_OK) return rc;
  const size_t pixels = (size_t)batch * oh * ow;
  // the im2col buffer (or, for a 1x1, the padded copy of the image rows) and the padded output, whether or not this
  // geometry and the run's pointers end up needing them
  if ((rc = h->col_ws.ensure(pixels * round_up(h->st.k, 16))) != MI_OK) return rc;
  return h->c_ws.ensure(pixels * round_up(h->st.n, 4));
}

int mi_conv_run(mi_conv *h, const int8_t *in_dev, int32_t batch, int32_t in_h, int32_t in_w, int8_t *out_dev,
                void *stream) {
  if (h == nullptr || in_dev == nullptr || out_dev == nullptr) {
    set_error("mi_conv_run: null argument");
    return MI_NULL_PTR;
  }
  if (batch < 0) return MI_PARAM_INVALID;
  int oh = 0, ow = 0;
  int rc = mi_conv_out_shape(h, in_h, in_w, &oh, &ow);
  if (rc != MI_OK) return rc;
  if (batch == 0) return MI_OK;
  if ((rc = ensure_device()) != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const mi_conv_desc &d = h->d;
  ConvGeom g{batch,       in_h,       in_w,       d.in_channel, oh,           ow,           d.out_channel, d.kernel_h,
             d.kernel_w,  d.stride_h, d.stride_w, d.dilation_h, d.dilation_w, d.pad_u,      d.pad_l};
  const int64_t pixels = (int64_t)batch * oh * ow;
  if (pixels > 0x7fffffff) {
    set_error("mi_conv_run: too many output pixels");
    return MI_PARAM_INVALID;
  }
  if (h->depthwise) {
    RequantParams rq = h->st.params();
    rq.fast = h->dw_fast ? 1 : 0;
    return launch_conv_dw(in_dev, g, static_cast<const int16_t *>(h->w16.p), static_cast<const int32_t *>(h->dw_bias.p),
                          static_cast<const int32_t *>(h->dw_bias_folded.p), (int)(int8_t)d.in_zp, rq, out_dev, s);
  }
  const int k = h->st.k;
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  if (h->direct_1x1) {
    if ((rc = prepare_rows(in_dev, (int)pixels, k, Workspace::growable(&h->col_ws), s, &a, &lda, &k16)) != MI_OK) return rc;
  } else if (k <= 64 && d.out_channel <= 128 && (d.out_channel & 3) == 0 &&
             (reinterpret_cast<uintptr_t>(out_dev) & 3) == 0) {
    // a first-layer convolution: gathered straight from the image, no im2col buffer
    return launch_conv_smallk(in_dev, g, h->fill, k, static_cast<const int8_t *>(h->st.w.p), h->st.ldw, h->st.params(),
                              out_dev, s);
  } else if (pixels > 128 && gemm_conv_supported(g, in_dev, out_dev)) {
    // 16-channel-aligned images: the GEMM gathers its activation operand from the image, no im2col buffer
    WeightView w{static_cast<const int8_t *>(h->st.w.p), h->st.k_pad, h->st.ldw, nullptr};
    return launch_gemm_conv_requant(in_dev, g, static_cast<const int8_t *>(h->fill16.p), w, h->st.params(), out_dev, s);
  } else {
    k16 = round_up(k, 16);
    if ((rc = h->col_ws.ensure((size_t)pixels * k16)) != MI_OK) return rc;
    if ((rc = launch_im2col(in_dev, g, h->fill, static_cast<int8_t *>(h->col_ws.p), k16, s)) != MI_OK) return rc;
    a = static_cast<const int8_t *>(h->col_ws.p);
    lda = k16;
  }
  return run_requant_gemm(h->st, a, lda, (int)pixels, k16, out_dev, Workspace::growable(&h->c_ws), s);
}

int mi_conv_run_host(mi_conv *h, const int8_t *in_host, int32_t batch, int32_t in_h, int32_t in_w, int8_t *out_host) {
  if (h == nullptr || in_host == nullptr || out_host == nullptr) {
    set_error("mi_conv_run_host: null argument");
    return MI_NULL_PTR;
  }
  int oh = 0, ow = 0;
  int rc = mi_conv_out_shape(h, in_h, in_w, &oh, &ow);
  if (rc != MI_OK) return rc;
  if (batch < 0) return MI_PARAM_INVALID;
  if (batch == 0) return MI_OK;
  if ((rc = ensure_device()) != MI_OK) return rc;
  const size_t in_bytes = (size_t)batch * in_h * in_w * h->d.in_channel;
  const size_t out_bytes = (size_t)batch * oh * ow * h->d.out_channel;
  if ((rc = h->h_in.ensure(in_bytes)) != MI_OK || (rc = h->h_out.ensure(out_bytes)) != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(h->h_in.p, in_host, in_bytes, hipMemcpyHostToDevice));
  rc = mi_conv_run(h, static_cast<const int8_t *>(h->h_in.p), batch, in_h, in_w, static_cast<int8_t *>(h->h_out.p),
                   nullptr);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(out_host, h->h_out.p, out_bytes, hipMemcpyDeviceToHost));
  return MI_OK;
}

void mi_conv_destroy(mi_conv *h) { delete h; }  // every DevBuf member frees its device memory

// ------------------------------------------------------------------------------------------------------- dynquant
int mi_dynquant_create(int32_t symmetric, mi_dynquant **out) {
  if (out == nullptr) return MI_NULL_PTR;
  *out = nullptr;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  std::unique_ptr<mi_dynquant> owner(new (std::nothrow) mi_dynquant());  // the buffers free themselves if anything below throws
  mi_dynquant *h = owner.get();
  if (h == nullptr) return MI_MEMORY_FAILED;
  h->symmetric = symmetric ? 1 : 0;
  if ((rc = h->partials.ensure(sizeof(float2) * kDqMaxBlocks)) != MI_OK ||
      (rc = h->params.ensure(sizeof(mi_dq_params))) != MI_OK) {
    return rc;
  }
  *out = owner.release();
  return MI_OK;
}

int mi_dynquant_run(mi_dynquant *h, const float *x_dev, int64_t n, int8_t *q_dev, void *stream) {
  if (h == nullptr || (n > 0 && (x_dev == nullptr || q_dev == nullptr))) {
    set_error("mi_dynquant_run: null argument");
    return MI_NULL_PTR;
  }
  if (n < 0) return MI_PARAM_INVALID;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  return launch_dynquant(x_dev, n, h->symmetric, static_cast<float2 *>(h->partials.p),
                         static_cast<mi_dq_params *>(h->params.p), q_dev, static_cast<hipStream_t>(stream));
}

int mi_dynquant_get_params(mi_dynquant *h, void *stream, mi_dq_params *params_host) {
  if (h == nullptr || params_host == nullptr) return MI_NULL_PTR;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  MI_HIP_CHECK(hipMemcpyAsync(params_host, h->params.p, sizeof(mi_dq_params), hipMemcpyDeviceToHost, s));
  MI_HIP_CHECK(counted_sync(s));
  return MI_OK;
}

int mi_dynquant_run_segments(mi_dynquant *h, const float *x_dev, int64_t segments, int64_t unit, int8_t *q_dev,
                             mi_dq_params *params_dev, void *stream) {
  if (h == nullptr || x_dev == nullptr || q_dev == nullptr || params_dev == nullptr) {
    set_error("mi_dynquant_run_segments: null argument");
    return MI_NULL_PTR;
  }
  if (segments < 1 || unit < 1) {
    set_error("mi_dynquant_run_segments: segments and unit must be positive");
    return MI_PARAM_INVALID;
  }
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  return launch_dynquant_segments(x_dev, segments, unit, h->symmetric, params_dev, q_dev,
                                  static_cast<hipStream_t>(stream));
}

int mi_dynquant_run_segments_host(mi_dynquant *h, const float *x_host, int64_t segments, int64_t unit, int8_t *q_host,
                                  mi_dq_params *params_host) {
  if (h == nullptr || x_host == nullptr || q_host == nullptr || params_host == nullptr) {
    set_error("mi_dynquant_run_segments_host: null argument");
    return MI_NULL_PTR;
  }
  if (segments < 1 || unit < 1) return MI_PARAM_INVALID;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  const size_t n = (size_t)segments * (size_t)unit;
  if ((rc = h->h_in.ensure(n * 4 + 16)) != MI_OK || (rc = h->h_out.ensure(n + 16)) != MI_OK ||
      (rc = h->h_params.ensure(sizeof(mi_dq_params) * (size_t)segments)) != MI_OK)
    return rc;
  MI_HIP_CHECK(hipMemcpy(h->h_in.p, x_host, n * 4, hipMemcpyHostToDevice));
  rc = mi_dynquant_run_segments(h, static_cast<const float *>(h->h_in.p), segments, unit,
                                static_cast<int8_t *>(h->h_out.p), static_cast<mi_dq_params *>(h->h_params.p), nullptr);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(q_host, h->h_out.p, n, hipMemcpyDeviceToHost));
  MI_HIP_CHECK(hipMemcpy(params_host, h->h_params.p, sizeof(mi_dq_params) * (size_t)segments, hipMemcpyDeviceToHost));
  return MI_OK;
}

const mi_dq_params *mi_dynquant_device_params(const mi_dynquant *h) {
  return h == nullptr ? nullptr : static_cast<const mi_dq_params *>(h->params.p);
}

int mi_dynquant_run_host(mi_dynquant *h, const float *x_host, int64_t n, int8_t *q_host, mi_dq_params *params_host) {
  if (h == nullptr || params_host == nullptr || (n > 0 && (x_host == nullptr || q_host == nullptr))) {
    set_error("mi_dynquant_run_host: null argument");
    return MI_NULL_PTR;
  }
  if (n < 0) return MI_PARAM_INVALID;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  if ((rc = h->h_in.ensure((size_t)n * 4 + 16)) != MI_OK || (rc = h->h_out.ensure((size_t)n + 16)) != MI_OK) return rc;
  if (n > 0) MI_HIP_CHECK(hipMemcpy(h->h_in.p, x_host, (size_t)n * 4, hipMemcpyHostToDevice));
  rc = mi_dynquant_run(h, static_cast<const float *>(h->h_in.p), n, static_cast<int8_t *>(h->h_out.p), nullptr);
  if (rc != MI_OK) return rc;
  if ((rc = mi_dynquant_get_params(h, nullptr, params_host)) != MI_OK) return rc;
  if (n > 0) MI_HIP_CHECK(hipMemcpy(q_host, h->h_out.p, (size_t)n, hipMemcpyDeviceToHost));
  return MI_OK;
}

void mi_dynquant_destroy(mi_dynquant *h) { delete h; }  // every DevBuf member frees its device memory

// ---------------------------------------------------------------------------------------------------------- dynmm
static int mi_dynmm_create_impl(const mi_dynmm_desc *d, const int8_t *weight_host, const float *bias_host, mi_dynmm **out) {
  if (d == nullptr || weight_host == nullptr || out == nullptr) {
    set_error("mi_dynmm_create: null argument");
    return MI_NULL_PTR;
  }
  *out = nullptr;
  if (d->deep <= 0 || d->col <= 0 || (d->act_type != MI_ACT_NONE && d->act_type != MI_ACT_RELU &&
                                      d->act_type != MI_ACT_RELU6)) {
    set_error("mi_dynmm_create: bad shape/activation");
    return MI_PARAM_INVALID;
  }
  if ((d->flags & ~(MI_DYNMM_WEIGHT_PACKED_SDOT | MI_DYNMM_NO_DECODE_PACK)) != 0) {
    set_error("mi_dynmm_create: unknown flags 0x%x", d->flags);
    return MI_PARAM_INVALID;
  }
  int rc = check_filter_quant(d->filter_quant_num, d->col, d->filter_scales, d->filter_zps);
  if (rc != MI_OK) return rc;
  if ((rc = ensure_device()) != MI_OK) return rc;
  std::unique_ptr<mi_dynmm> owner(new (std::nothrow) mi_dynmm());  // the buffers free themselves if anything below throws
  mi_dynmm *h = owner.get();
  if (h == nullptr) return MI_MEMORY_FAILED;
  h->n = d->col;
  h->k = d->deep;
  h->n_pad = round_up(h->n, kNPad);
  h->k_pad = round_up(h->k, kKPad);
  h->ldw = weight_row_stride(h->k_pad);
  h->act = d->act_type;
  h->zw0 = d->filter_zps[0];
  h->has_bias = bias_host != nullptr;
  const bool packed_sdot = (d->flags & MI_DYNMM_WEIGHT_PACKED_SDOT) != 0;
  const std::vector<int8_t> w_nk = packed_sdot ? unpack_4x16(weight_host, h->n, h->k)
                                               : to_nk(weight_host, h->n, h->k, d->b_transpose);
  std::vector<int8_t> packed((size_t)h->n_pad * h->ldw, 0);
  std::vector<float> ws(h->n_pad, 0.0f), bs(h->n_pad, 0.0f);
  std::vector<int32_t> wsum(h->n_pad, 0);
  for (int c = 0; c < h->n; ++c) {
    memcpy(packed.data() + (size_t)c * h->ldw, w_nk.data() + (size_t)c * h->k, (size_t)h->k);
    int32_t s = 0;
    for (int i = 0; i < h->k; ++i) s += w_nk[(size_t)c * h->k + i];
    // a model that carries its own weight sums is computed with those (matmul_dynamic_base_int8.cc:179-183)
    wsum[c] = (packed_sdot && d->weight_sums != nullptr) ? d->weight_sums[c] : s;
    ws[c] = (float)d->filter_scales[d->filter_quant_num > 1 ? c : 0];
    if (bias_host != nullptr) bs[c] = bias_host[c];
  }
  rc = upload(&h->w, packed);
  if (rc == MI_OK) rc = upload(&h->wscale, ws);
  if (rc == MI_OK) rc = upload(&h->wsum, wsum);
  if (rc == MI_OK && h->has_bias) rc = upload(&h->bias, bs);
  if (rc != MI_OK) {
    return rc;
  }
  if ((d->flags & MI_DYNMM_NO_DECODE_PACK) == 0) {
    // as for mi_matmul: an optimisation for few activation rows (decode), not a requirement -- without it those row
    // counts run on the GEMM tiles, and a device without room for the copy still gets a working handle
    rc = h->w_blocked.ensure((size_t)h->n_pad * h->k_pad);
    if (rc == MI_OK)
      rc = launch_block_weights(static_cast<const int8_t *>(h->w.p), h->n_pad, h->k_pad, h->ldw,
                                static_cast<int8_t *>(h->w_blocked.p), nullptr);
    if (rc == MI_OK && hipStreamSynchronize(nullptr) != hipSuccess) rc = MI_ERROR;
    if (rc != MI_OK) {
      (void)hipGetLastError();
      h->w_blocked.release();
      set_error("");
    }
  }
  *out = owner.release();
  return MI_OK;
}

int mi_unpack_weight_4x16(const int8_t *packed, int32_t col, int32_t deep, int8_t *weight_nk) {
  if (packed == nullptr || weight_nk == nullptr) return MI_NULL_PTR;
  if (col <= 0 || deep <= 0) return MI_PARAM_INVALID;
  return guarded("mi_unpack_weight_4x16", [&] {
    const std::vector<int8_t> w = unpack_4x16(packed, col, deep);
    memcpy(weight_nk, w.data(), w.size());
    return MI_OK;
  });
}

int mi_dynmm_create(const mi_dynmm_desc *d, const int8_t *weight_host, const float *bias_host, mi_dynmm **out) {
  return guarded("mi_dynmm_create", [&] { return mi_dynmm_create_impl(d, weight_host, bias_host, out); });
}

static DequantParams dequant_params(const mi_dynmm *h, float sx, int32_t zx, const mi_dq_params *qp_dev, bool per_row) {
  DequantParams dq;
  dq.wscale = static_cast<const float *>(h->wscale.p);
  dq.bias = h->has_bias ? static_cast<const float *>(h->bias.p) : nullptr;
  dq.wsum = static_cast<const int32_t *>(h->wsum.p);
  dq.qp_dev = qp_dev;
  dq.sx = sx;
  dq.zx = zx;
  dq.zw0 = h->zw0;
  dq.per_row = per_row ? 1 : 0;
  dq.deep = h->k;
  dq.act = h->act;
  return dq;
}

static int dynmm_run_impl(mi_dynmm *h, const int8_t *a_dev, int32_t rows, float sx, int32_t zx,
                          const mi_dq_params *qp_dev, float *c_dev, hipStream_t s, bool per_row = false) {
  if (h == nullptr || a_dev == nullptr || c_dev == nullptr) {
    set_error("mi_dynmm_run: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) return MI_PARAM_INVALID;
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  if ((rc = prepare_rows(a_dev, rows, h->k, Workspace::growable(&h->a_ws), s, &a, &lda, &k16)) != MI_OK) return rc;
  const DequantParams dq = dequant_params(h, sx, zx, qp_dev, per_row);
  const WeightView w{static_cast<const int8_t *>(h->w.p), h->k_pad, h->ldw,
                     static_cast<const int8_t *>(h->w_blocked.p)};
  // decode-sized runs: the matrix-core decode kernel streams the blocked weights once (any N, any output alignment)
  // (one row runs on the row-major weights and needs no blocked copy, as long as the row fits the kernel's LDS form)
  if (gemv_takes_rows(rows, h->n, h->k_pad) && (rows > kGemvDotRows || (int64_t)rows * k16 <= 150 * 1024) &&
      (rows == 1 || (w.blocked != nullptr && h->k_pad <= 1 << 20)))
    return launch_gemv_dequant(a, lda, rows, k16, w, h->n, dq, c_dev, h->n, s);
  if ((h->n & 3) == 0 && (reinterpret_cast<uintptr_t>(c_dev) & 15) == 0)
    return launch_gemm_dequant(a, lda, rows, k16, w, h->n, dq, c_dev, h->n, s);
  const int n4 = round_up(h->n, 4);
  if ((rc = h->c_ws.ensure((size_t)rows * n4 * sizeof(float))) != MI_OK) return rc;
  if ((rc = launch_gemm_dequant(a, lda, rows, k16, w, n4, dq, static_cast<float *>(h->c_ws.p), n4, s)) != MI_OK)
    return rc;
  return launch_copy_rows(h->c_ws.p, (int64_t)n4 * 4, rows, h->n * 4, c_dev, (int64_t)h->n * 4, s);
}

int mi_dynmm_reserve(mi_dynmm *h, int32_t max_rows) {
  if (h == nullptr) return MI_NULL_PTR;
  if (max_rows < 0) return MI_PARAM_INVALID;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  if ((rc = h->a_ws.ensure((size_t)max_rows * round_up(h->k, 16))) != MI_OK) return rc;
  return h->c_ws.ensure((size_t)max_rows * round_up(h->n, 4) * sizeof(float));
}

int mi_dynmm_run(mi_dynmm *h, const int8_t *a_dev, int32_t rows, double in_scale, int32_t in_zp, float *c_dev,
                 void *stream) {
  return dynmm_run_impl(h, a_dev, rows, (float)in_scale, in_zp, nullptr, c_dev, static_cast<hipStream_t>(stream));
}

int mi_dynmm_run_chained(mi_dynmm *h, const int8_t *a_dev, int32_t rows, const mi_dq_params *params_dev, float *c_dev,
                         void *stream) {
  if (params_dev == nullptr) {
    set_error("mi_dynmm_run_chained: params_dev is null");
    return MI_NULL_PTR;
  }
  return dynmm_run_impl(h, a_dev, rows, 0.0f, 0, params_dev, c_dev, static_cast<hipStream_t>(stream));
}

int mi_dynmm_run_rows(mi_dynmm *h, const int8_t *a_dev, int32_t rows, const mi_dq_params *row_params_dev, float *c_dev,
                      void *stream) {
  if (row_params_dev == nullptr) {
    set_error("mi_dynmm_run_rows: row_params_dev is null");
    return MI_NULL_PTR;
  }
  return dynmm_run_impl(h, a_dev, rows, 0.0f, 0, row_params_dev, c_dev, static_cast<hipStream_t>(stream), true);
}

int mi_dynmm_run_group(mi_dynmm *const *handles, int32_t count, const int8_t *a_dev, int32_t rows, double in_scale,
                       int32_t in_zp, const mi_dq_params *params_dev, int32_t per_row, float *const *c_dev,
                       void *stream) {
  if (handles == nullptr || a_dev == nullptr || c_dev == nullptr) {
    set_error("mi_dynmm_run_group: null argument");
    return MI_NULL_PTR;
  }
  if (count < 1 || rows < 0 || (per_row != 0 && params_dev == nullptr)) {
    set_error("mi_dynmm_run_group: count=%d rows=%d per_row=%d", count, rows, per_row);
    return MI_PARAM_INVALID;
  }
  for (int i = 0; i < count; ++i) {
    if (handles[i] == nullptr || c_dev[i] == nullptr) {
      set_error("mi_dynmm_run_group: member %d is null", i);
      return MI_NULL_PTR;
    }
    if (handles[i]->k != handles[0]->k) {
      set_error("mi_dynmm_run_group: member %d has deep=%d, member 0 has %d", i, handles[i]->k, handles[0]->k);
      return MI_PARAM_INVALID;
    }
  }
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int8_t *a = nullptr;
  int64_t lda = 0;
  int k16 = 0;
  // the activation rows are brought into the kernels' form once, for all members
  if ((rc = prepare_rows(a_dev, rows, handles[0]->k, Workspace::growable(&handles[0]->a_ws), s, &a, &lda, &k16)) != MI_OK)
    return rc;
  // decode-sized runs of up to four members go out as one launch; anything else runs member by member
  bool one_launch = count >= 2 && count <= 4 && rows <= kGemvGroupMaxRows &&
                    (rows > kGemvDotRows || (int64_t)rows * k16 <= 150 * 1024);
  for (int i = 0; i < count && one_launch; ++i)
    one_launch = rows == 1 || (handles[i]->w_blocked.p != nullptr && handles[i]->k_pad <= 1 << 20);
  if (one_launch) {
    WeightView wv[4];
    DequantParams dq[4];
    int n[4];
    for (int i = 0; i < count; ++i) {
      const mi_dynmm *h = handles[i];
      wv[i] = WeightView{static_cast<const int8_t *>(h->w.p), h->k_pad, h->ldw, static_cast<const int8_t *>(h->w_blocked.p)};
      dq[i] = dequant_params(h, (float)in_scale, in_zp, params_dev, per_row != 0);
      n[i] = h->n;
    }
    return launch_gemv_group_dequant(a, lda, rows, k16, count, wv, n, dq, c_dev, s);
  }
  for (int i = 0; i < count; ++i) {
    if ((rc = dynmm_run_impl(handles[i], a_dev, rows, (float)in_scale, in_zp, params_dev, c_dev[i], s, per_row != 0)) != MI_OK)
      return rc;
  }
  return MI_OK;
}

static int mi_dynmm_run_rows_host_impl(mi_dynmm *h, const int8_t *a_host, int32_t rows, const double *in_scales, int32_t in_zp,
                           float *c_host) {
  if (h == nullptr || a_host == nullptr || c_host == nullptr || in_scales == nullptr) {
    set_error("mi_dynmm_run_rows_host: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) return MI_PARAM_INVALID;
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  const size_t in_bytes = (size_t)rows * h->k, out_bytes = (size_t)rows * h->n * sizeof(float);
  if ((rc = h->h_in.ensure(in_bytes)) != MI_OK || (rc = h->h_out.ensure(out_bytes)) != MI_OK ||
      (rc = h->h_params.ensure(sizeof(mi_dq_params) * (size_t)rows)) != MI_OK)
    return rc;
  std::vector<mi_dq_params> p((size_t)rows);
  for (int r = 0; r < rows; ++r) {
    p[r].scale = in_scales[r];
    p[r].scale_f = (float)in_scales[r];  // the wrapper narrows every input scale to float (matmul_dynamic_base_int8.cc:168-171)
    p[r].zero_point = in_zp;
    p[r].real_min = p[r].real_max = 0.0f;
  }
  MI_HIP_CHECK(hipMemcpy(h->h_params.p, p.data(), sizeof(mi_dq_params) * (size_t)rows, hipMemcpyHostToDevice));
  MI_HIP_CHECK(hipMemcpy(h->h_in.p, a_host, in_bytes, hipMemcpyHostToDevice));
  rc = mi_dynmm_run_rows(h, static_cast<const int8_t *>(h->h_in.p), rows,
                         static_cast<const mi_dq_params *>(h->h_params.p), static_cast<float *>(h->h_out.p), nullptr);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(c_host, h->h_out.p, out_bytes, hipMemcpyDeviceToHost));
  return MI_OK;
}

int mi_dynmm_run_rows_host(mi_dynmm *h, const int8_t *a_host, int32_t rows, const double *in_scales, int32_t in_zp,
                           float *c_host) {
  return guarded("mi_dynmm_run_rows_host", [&] { return mi_dynmm_run_rows_host_impl(h, a_host, rows, in_scales, in_zp, c_host); });
}

int mi_dynmm_run_host(mi_dynmm *h, const int8_t *a_host, int32_t rows, double in_scale, int32_t in_zp, float *c_host) {
  if (h == nullptr || a_host == nullptr || c_host == nullptr) {
    set_error("mi_dynmm_run_host: null argument");
    return MI_NULL_PTR;
  }
  if (rows < 0) return MI_PARAM_INVALID;
  if (rows == 0) return MI_OK;
  int rc = ensure_device();
  if (rc != MI_OK) return rc;
  const size_t in_bytes = (size_t)rows * h->k, out_bytes = (size_t)rows * h->n * sizeof(float);
  if ((rc = h->h_in.ensure(in_bytes)) != MI_OK || (rc = h->h_out.ensure(out_bytes)) != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(h->h_in.p, a_host, in_bytes, hipMemcpyHostToDevice));
  rc = mi_dynmm_run(h, static_cast<const int8_t *>(h->h_in.p), rows, in_scale, in_zp, static_cast<float *>(h->h_out.p),
                    nullptr);
  if (rc != MI_OK) return rc;
  MI_HIP_CHECK(hipMemcpy(c_host, h->h_out.p, out_bytes, hipMemcpyDeviceToHost));
  return MI_OK;
}

void mi_dynmm_destroy(mi_dynmm *h) { delete h; }  // every DevBuf member frees its device memory

}  // extern "C"
