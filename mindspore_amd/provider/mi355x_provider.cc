// MindSpore Lite custom-provider kernels backed by libmi355x_int8.so.
//
// This translation unit is the reference-side half of the drop-in boundary: it subclasses mindspore::kernel::Kernel
// (include/api/kernel.h:29-55) and registers creators through registry::RegisterKernel
// (mindspore/lite/include/registry/register_kernel.h:57-74) for MatMulFusion, FullConnection, Conv2DFusion (int8) and
// DynamicQuant (float32).  Everything below the Kernel objects is the C ABI of include/mi355x_int8.h.
//
// No kernel::KernelInterface is registered for these operator types, on purpose.  They are builtin types: when a
// provider's interface answers, Scheduler::InferNodeShape returns before it creates the node's OpParameter
// (mindspore/lite/src/litert/scheduler.cc:652-698), and a node that a creator below then declines can no longer fall
// back to the builtin kernel (FindBackendKernel finds no OpParameter, :1178-1183) -- Model::Build would fail for
// every fp32 convolution of the graph.  The builtin inference produces the same shapes (and the data types), and
// ConvKernel::ReSize derives SAME-mode padding from the tensor shapes itself.
//
// It needs a MindSpore Lite SDK to compile (register_kernel.h includes the flatc-generated schema/model_generated.h)
// and is therefore not part of the library build:
//   g++ -std=c++17 -fPIC -shared mi355x_provider.cc -I<lite-sdk>/runtime -I<repo>/include
//       -L<lite-sdk>/runtime/lib -lmindspore-lite -L<repo>/mindspore_amd -lmi355x_int8 -o libmi355x_provider.so
// Without an SDK the tests compile it against hand-written stand-ins of those headers (tests/lite_stub) and drive it
// through a harness that plays the scheduler.
// An application selects it with CPUDeviceInfo::SetProvider("mi355x") (+ SetProviderDevice("CPU")); the stock
// benchmark tool with --provider=mi355x (it leaves the provider device empty, hence the second registration under "").
//
// Tensors are host-resident (arch "CPU": the kernels live in the ordinary CPU subgraph).  Every kernel computes into
// a device buffer of its own, publishes that address on its output tensor (MSTensor::SetDeviceData,
// include/api/types.h:295-305) and copies the result to the tensor's host memory; a kernel whose input carries an
// address published by another kernel of this provider reads it in place and skips the upload.  The session config
//   [mi355x]
//   device_only_outputs=<tensor name>,<tensor name>,...      (or * for every output)
// (Model::LoadConfig / UpdateConfig, delivered through Kernel::GetConfig, include/api/kernel_api.h:112-126) names
// outputs that only kernels of this provider consume: their host copy is skipped as well.
// Dense 3x3 stride-1 convolutions are declined by default: x86 builds of the reference run an integer Winograd there
// (convolution_int8_creator.cc:81-94), whose results are not those of the exact convolution.  MI355X_CONV3X3=exact in
// the environment makes the provider take them and compute the exact convolution, which is what the reference runs
// on ARM64 cores with dot-product instructions -- for models validated on such devices.
// A creator returns nullptr for everything the library does not reproduce bit-exactly; the scheduler then falls back
// to the builtin CPU kernel (mindspore/lite/src/litert/scheduler.cc:1173-1177).
#include <stdlib.h>

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "include/api/kernel.h"
#include "include/api/status.h"
#include "include/api/types.h"
#include "include/registry/register_kernel.h"
#include "mi355x_int8.h"
#include "schema/model_generated.h"

namespace mindspore {
namespace mi355x {
namespace {
constexpr int kWeightIndex = 1;
constexpr int kBiasIndex = 2;

// The GPU the provider runs on: HIP device 0, or the one MI355X_DEVICE names (a CPUDeviceInfo has no device id).
bool LibraryReady() {
  static const bool ok = [] {
    const char *device = getenv("MI355X_DEVICE");
    return mi_init(device != nullptr ? atoi(device) : 0) == MI_OK;
  }();
  return ok;
}

// A creator cannot see the session config (the scheduler hands it over after creation), hence the environment.
bool Exact3x3() {
  const char *v = getenv("MI355X_CONV3X3");
  return v != nullptr && std::string(v) == "exact";
}

// Per-tensor activation quantisation is all the builtin kernels accept too (convolution_base.cc:334-342,368-375).
bool PerTensor(const MSTensor &t) { return t.QuantParams().size() == 1; }

void FilterQuant(const MSTensor &w, std::vector<double> *scales, std::vector<int32_t> *zps) {
  for (const auto &q : w.QuantParams()) {
    scales->push_back(q.scale);
    zps->push_back(q.zero_point);
  }
}

int ToStatus(int mi_code) { return mi_code == MI_OK ? static_cast<int>(kSuccess) : static_cast<int>(kLiteError); }

}  // namespace

// One HIP stream per session: every kernel of a session is handed the same mindspore::Context, and everything it
// launches or copies goes to that session's stream, so that sessions running on different threads neither share a
// queue nor wait for each other's copies.  A provider is never told that a session ended, so the stream is counted:
// every kernel takes a reference in Prepare and gives it back when it is destroyed, and the last one destroys the
// stream (its own work on it has finished by then: a kernel's buffers are freed first, which waits for the device).
class SessionStreams {
 public:
  static void *Acquire(const Context *ctx) {
    std::lock_guard<std::mutex> lock(Mutex());
    Entry &e = Map()[ctx];
    if (e.refs == 0 && mi_stream_create(&e.stream) != MI_OK) e.stream = nullptr;  // the null stream still works, only without overlap
    ++e.refs;
    return e.stream;
  }
  static void Release(const Context *ctx) {
    std::lock_guard<std::mutex> lock(Mutex());
    auto it = Map().find(ctx);
    if (it == Map().end() || --it->second.refs > 0) return;
    mi_stream_destroy(it->second.stream);
    Map().erase(it);
  }
  static size_t Count() {
    std::lock_guard<std::mutex> lock(Mutex());
    return Map().size();
  }

 private:
  struct Entry {
    void *stream = nullptr;
    int refs = 0;
  };
  static std::mutex &Mutex() {
    static std::mutex *m = new std::mutex;
    return *m;
  }
  static std::map<const Context *, Entry> &Map() {
    static auto *m = new std::map<const Context *, Entry>;
    return *m;
  }
};

// Rows of a MatMul / FullConnection: the product of the output's leading dimensions, as the reference kernels take
// it (fullconnection_int8.cc:49-58, which also covers use_axis; matmul_int8.cc InitParameter).
int64_t RowsOfOutput(const MSTensor &out) {
  const auto shape = out.Shape();
  int64_t rows = 1;
  for (size_t i = 0; i + 1 < shape.size(); ++i) rows *= shape[i];
  return rows;
}

// Device addresses this provider has published on tensors.  GetDeviceData() of an input is trusted only when it is
// one of them: an application may have attached memory of some other device to a graph input.
// Each address also carries a version, counted up whenever its owner delivers a new result into it, and -- for the
// output of a DynamicQuant kernel -- where that run's scales and zero points lie in device memory.
struct QuantOnDevice {
  const mi_dq_params *params = nullptr;  // one block (per tensor), or one per row
  bool per_row = false;
  int64_t rows = 0;
};

class Published {
 public:
  static void Add(void *p) {
    std::lock_guard<std::mutex> lock(Mutex());
    (void)Table()[p];
  }
  static void Remove(void *p) {
    std::lock_guard<std::mutex> lock(Mutex());
    Table().erase(p);
  }
  static bool Has(void *p) {
    std::lock_guard<std::mutex> lock(Mutex());
    return Table().count(p) != 0;
  }
  // a new result was written into p (its owner's Deliver)
  static void Bump(void *p, const QuantOnDevice *quant) {
    std::lock_guard<std::mutex> lock(Mutex());
    auto it = Table().find(p);
    if (it == Table().end()) return;
    ++it->second.version;
    it->second.quant = quant != nullptr ? *quant : QuantOnDevice{};
  }
  // 0 for an address that is not one of this provider's
  static int64_t Version(void *p) {
    std::lock_guard<std::mutex> lock(Mutex());
    auto it = Table().find(p);
    return it == Table().end() ? 0 : it->second.version;
  }
  static bool Quant(void *p, QuantOnDevice *out) {
    std::lock_guard<std::mutex> lock(Mutex());
    auto it = Table().find(p);
    if (it == Table().end() || it->second.quant.params == nullptr) return false;
    *out = it->second.quant;
    return true;
  }

 private:
  struct Entry {
    int64_t version = 1;
    QuantOnDevice quant;
  };
  // never destroyed: kernels owned by a session with static storage may be torn down after this file's statics
  static std::mutex &Mutex() {
    static std::mutex *m = new std::mutex;
    return *m;
  }
  static std::unordered_map<void *, Entry> &Table() {
    static auto *t = new std::unordered_map<void *, Entry>;
    return *t;
  }
};

// Device memory a kernel owns; grows, never shrinks.
class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  ~DeviceBuffer() { Release(); }
  void *Reserve(size_t bytes) {
    if (bytes > cap_) {
      Release();
      if (mi_device_malloc(bytes, &p_) != MI_OK) return nullptr;
      cap_ = bytes;
    }
    return p_;
  }
  void *get() const { return p_; }
  void Release() {
    if (p_ != nullptr) {
      Published::Remove(p_);
      mi_device_free(p_);
    }
    p_ = nullptr;
    cap_ = 0;
  }

 private:
  void *p_ = nullptr;
  size_t cap_ = 0;
};

// What every kernel of this provider does around its launch: find input 0 on the device (in place when a kernel of
// this provider left it there, uploaded otherwise) and hand the output on.
class DeviceIo {
 public:
  DeviceIo() = default;
  DeviceIo(const DeviceIo &) = delete;
  DeviceIo &operator=(const DeviceIo &) = delete;
  ~DeviceIo() {
    in_.Release();  // (waits for the device: nothing of this kernel is left on the stream)
    out_.Release();
    if (configured_) SessionStreams::Release(ctx_);
  }

  // the session's stream, and [mi355x] device_only_outputs for the given output tensor
  void Configure(const Context *ctx, const std::map<std::string, std::string> &section, const std::string &output_name) {
    if (!configured_) {
      ctx_ = ctx;
      stream_ = SessionStreams::Acquire(ctx);
      configured_ = true;
    }
    const auto it = section.find("device_only_outputs");
    if (it == section.end()) return;
    const std::string &list = it->second;
    size_t pos = 0;
    while (pos <= list.size()) {
      size_t end = list.find(',', pos);
      if (end == std::string::npos) end = list.size();
      size_t b = pos, e = end;
      while (b < e && list[b] == ' ') ++b;
      while (e > b && list[e - 1] == ' ') --e;
      const std::string name = list.substr(b, e - b);
      if (name == "*" || (!name.empty() && name == output_name)) host_copy_ = false;
      pos = end + 1;
    }
  }

  const void *Input(MSTensor *t) {
    void *dev = t->GetDeviceData();
    if (dev != nullptr && Published::Has(dev)) return dev;
    const auto host = t->Data();
    const size_t bytes = t->DataSize();
    if (host == nullptr || bytes == 0) return nullptr;
    void *staged = in_.Reserve(bytes);
    // (returns once the bytes have left the host buffer: the runtime may recycle it as soon as Execute returns)
    if (staged == nullptr || mi_copy_to_device(staged, host.get(), bytes, stream_) != MI_OK) return nullptr;
    return staged;
  }

  void *Output(size_t bytes) {
    void *p = out_.Reserve(bytes);
    if (p != nullptr) Published::Add(p);
    return p;
  }

  // after the launch: publish the device address; copy to the host unless the output was declared device-only (the
  // copy waits for this session's stream only; a device-only output is ordered by the stream itself)
  int Deliver(MSTensor *t, const QuantOnDevice *quant = nullptr) {
    Published::Bump(out_.get(), quant);
    t->SetDeviceData(out_.get());
    if (!host_copy_) return kSuccess;
    void *host = t->MutableData();
    if (host == nullptr) return kLiteNullptr;
    return mi_copy_to_host(host, out_.get(), t->DataSize(), stream_) == MI_OK ? static_cast<int>(kSuccess)
                                                                               : static_cast<int>(kLiteError);
  }
  void *stream() const { return stream_; }
  bool host_copy() const { return host_copy_; }

  void Withdraw(MSTensor *t) {
    if (t->GetDeviceData() == out_.get()) t->SetDeviceData(nullptr);
  }

 private:
  DeviceBuffer in_, out_;
  bool host_copy_ = true;
  void *stream_ = nullptr;
  const Context *ctx_ = nullptr;
  bool configured_ = false;
};

// ---- MatMulFusion / FullConnection, int8 in -> int8 out (full quant) or fp32 out (dynamic quant) ----------------
class MatmulKernel;

// Full-quant MatMuls of one session that read the same input tensor with the same K (the gate and up projections of
// a decoder layer, q / k / v when they are separate nodes).  With a few activation rows each of them is a launch of a
// few microseconds whose fixed part is a fifth of it, so the first member that the session executes runs all of them
// as one launch (mi_matmul_run_group) and the others find their result waiting.  This leans on what a Lite session
// does (sub_graph_kernel.cc:456-466): the nodes of a graph are executed one after the other, each once per run, in
// the same order every run, and a tensor has one producer, so between the first sibling's Execute and the last one's
// nobody writes the shared input.  Sessions with Context::SetEnableParallel(true) form no groups.
std::atomic<int64_t> g_group_launches{0};

class SiblingGroup {
 public:
  static constexpr size_t kMaxMembers = 4;  // what mi_matmul_run_group takes as one launch
  static std::shared_ptr<SiblingGroup> Join(const Context *ctx, const MSTensor &input, int32_t k, MatmulKernel *m) {
    std::lock_guard<std::mutex> lock(Mutex());
    auto &groups = Groups();
    for (auto it = groups.begin(); it != groups.end();) {
      auto grp = it->lock();
      if (grp == nullptr) {
        it = groups.erase(it);
        continue;
      }
      if (grp->ctx_ == ctx && grp->k_ == k && grp->input_ == input && grp->members_.size() < kMaxMembers) {
        grp->members_.push_back(m);
        return grp;
      }
      ++it;
    }
    auto grp = std::make_shared<SiblingGroup>(ctx, input, k);
    grp->members_.push_back(m);
    groups.push_back(grp);
    return grp;
  }
  SiblingGroup(const Context *ctx, const MSTensor &input, int32_t k) : ctx_(ctx), input_(input), k_(k) {}
  void Leave(MatmulKernel *m) {
    std::lock_guard<std::mutex> lock(Mutex());
    for (auto it = members_.begin(); it != members_.end(); ++it) {
      if (*it == m) {
        members_.erase(it);
        break;
      }
    }
  }
  // (members of one session run on that session's thread; the lock only guards joining and leaving)
  std::vector<MatmulKernel *> Members() {
    std::lock_guard<std::mutex> lock(Mutex());
    return members_;
  }

 private:
  static std::mutex &Mutex() {
    static std::mutex *m = new std::mutex;
    return *m;
  }
  static std::vector<std::weak_ptr<SiblingGroup>> &Groups() {
    static auto *g = new std::vector<std::weak_ptr<SiblingGroup>>;
    return *g;
  }
  const Context *ctx_;
  MSTensor input_;  // a handle on the shared tensor object
  int32_t k_;
  std::vector<MatmulKernel *> members_;
};

class MatmulKernel : public kernel::Kernel {
 public:
  MatmulKernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const schema::Primitive *prim,
               const Context *ctx, bool b_transpose, int act)
      : Kernel(in, out, prim, ctx), b_transpose_(b_transpose), act_(act) {}
  ~MatmulKernel() override {
    if (group_ != nullptr) group_->Leave(this);
    io_.Withdraw(&outputs_[0]);
    mi_matmul_destroy(full_);
    mi_dynmm_destroy(dyn_);
  }

  int Prepare() override {
    io_.Configure(context_, GetConfig("mi355x"), outputs_[0].Name());
    const MSTensor &w = inputs_[kWeightIndex];
    const auto wshape = w.Shape();
    if (wshape.size() < 2 || w.Data() == nullptr) return kLiteError;
    const size_t r = wshape.size();
    const int32_t n = static_cast<int32_t>(b_transpose_ ? wshape[r - 2] : wshape[r - 1]);
    const int32_t k = static_cast<int32_t>(b_transpose_ ? wshape[r - 1] : wshape[r - 2]);
    k_ = k;
    n_ = n;
    int64_t b_batch = 1;  // a constant weight of rank > 2 is a batch of matrices (matmul_base_int8.cc:366-368)
    for (size_t i = 0; i + 2 < r; ++i) b_batch *= wshape[i];
    batched_ = r > 2;
    std::vector<double> scales;
    std::vector<int32_t> zps;
    FilterQuant(w, &scales, &zps);
    const void *bias = inputs_.size() > kBiasIndex ? inputs_[kBiasIndex].Data().get() : nullptr;
    // The second packed form of the weights serves up to 64 activation rows; a node whose inferred output already has
    // more rows than that does without it (half the device memory per weight).  Should the model later be resized
    // to a few rows, they run on the GEMM tiles.
    const auto oshape = outputs_[0].Shape();
    bool rows_known = !oshape.empty();
    for (int64_t e : oshape) rows_known = rows_known && e >= 0;
    const int64_t rows_now = batched_ && oshape.size() >= 2 ? oshape[oshape.size() - 2] : RowsOfOutput(outputs_[0]);
    const bool no_decode_pack = rows_known && rows_now > (n <= 4096 && k >= 1024 ? 2 * kDecodeMaxRows : kDecodeMaxRows);
    if (outputs_[0].DataType() == DataType::kNumberTypeInt8) {
      const auto iq = inputs_[0].QuantParams().front();
      const auto oq = outputs_[0].QuantParams().front();
      mi_matmul_desc d{k, n, b_transpose_ ? 1 : 0, act_, iq.scale, iq.zero_point, oq.scale, oq.zero_point,
                       static_cast<int32_t>(scales.size()), scales.data(), zps.data()};
      d.b_batch = static_cast<int32_t>(b_batch);
      if (no_decode_pack) d.flags |= MI_MATMUL_NO_DECODE_PACK;
      const int rc = mi_matmul_create(&d, static_cast<const int8_t *>(w.Data().get()),
                                      static_cast<const int32_t *>(bias), &full_);
      // (a session that runs its nodes in parallel gives no order to lean on: no groups there)
      if (rc == MI_OK && !batched_ && !inputs_[0].IsConst() && context_ != nullptr && !context_->GetEnableParallel() &&
          getenv("MI355X_NO_SIBLING_GROUPS") == nullptr) {
        group_ = SiblingGroup::Join(context_, inputs_[0], k, this);
      }
      return ToStatus(rc);
    }
    if (batched_) return kLiteError;  // (the creator declines batched weights for the dynamic MatMul)
    mi_dynmm_desc d{k, n, b_transpose_ ? 1 : 0, act_, static_cast<int32_t>(scales.size()), scales.data(), zps.data()};
    if (no_decode_pack) d.flags |= MI_DYNMM_NO_DECODE_PACK;
    const int rc =
      mi_dynmm_create(&d, static_cast<const int8_t *>(w.Data().get()), static_cast<const float *>(bias), &dyn_);
    // dynamic MatMuls that read the same DynamicQuant output (q / k / v, gate / up) form groups like the full-quant ones
    if (rc == MI_OK && !inputs_[0].IsConst() && context_ != nullptr && !context_->GetEnableParallel() &&
        getenv("MI355X_NO_SIBLING_GROUPS") == nullptr) {
      group_ = SiblingGroup::Join(context_, inputs_[0], k, this);
    }
    return ToStatus(rc);
  }

  int ReSize() override {  // the row count is read from the input tensor at every Execute
    computed_by_sibling_ = false;
    return kSuccess;
  }

  int Execute() override {
    if (batched_) return ExecuteBatched();
    const int32_t rows = static_cast<int32_t>(RowsOfOutput(outputs_[0]));
    if (rows == 0) return kSuccess;
    if (inputs_[0].ElementNum() != static_cast<int64_t>(rows) * k_) return kLiteError;
    if (computed_by_sibling_) {
      // A sibling's launch wrote this kernel's output buffer, on the session's stream.  It is this run's result if
      // the input is still the memory the sibling read -- and, where a kernel of this provider produces the input,
      // still the version it read (a producer counts its deliveries).  Where the producer is a builtin kernel the
      // order of a Lite session is what is left to lean on: siblings execute in the same run as the member that
      // launched for them.  MI355X_NO_SIBLING_GROUPS=1 in the environment switches the grouping off.
      computed_by_sibling_ = false;
      if (sibling_rows_ == rows && sibling_host_ == inputs_[0].Data().get() &&
          sibling_dev_ == inputs_[0].GetDeviceData() && sibling_version_ == Published::Version(sibling_dev_)) {
        return io_.Deliver(&outputs_[0]);
      }
    }
    if (group_ != nullptr && rows <= kSiblingMaxRows) {
      const int rc = ExecuteWithSiblings(rows);
      if (rc != kNotGrouped) return rc;
    }
    const auto *a = static_cast<const int8_t *>(io_.Input(&inputs_[0]));
    void *c = io_.Output(outputs_[0].DataSize());
    if (a == nullptr || c == nullptr) return kLiteNullptr;
    int rc = MI_ERROR;
    QuantOnDevice on_dev;
    if (full_ != nullptr) {
      rc = mi_matmul_run(full_, a, rows, static_cast<int8_t *>(c), io_.stream());
    } else if (a == inputs_[0].GetDeviceData() && Published::Quant(const_cast<int8_t *>(a), &on_dev) &&
               (!on_dev.per_row || on_dev.rows == rows)) {
      // the input was left on the device by this provider's DynamicQuant kernel, and so were its scale and zero
      // point (one block, or one per row): they are read there, in stream order, and the host has nothing to wait for
      rc = on_dev.per_row ? mi_dynmm_run_rows(dyn_, a, rows, on_dev.params, static_cast<float *>(c), io_.stream())
                          : mi_dynmm_run_chained(dyn_, a, rows, on_dev.params, static_cast<float *>(c), io_.stream());
    } else {
      // dynamic quant: the input's scale and zero point were written by the preceding DynamicQuant kernel during
      // this very inference, so they are read now, not in Prepare (matmul_dynamic_base_int8.cc:146-176)
      const auto iqs = inputs_[0].QuantParams();
      if (iqs.size() == 1) {
        rc = mi_dynmm_run(dyn_, a, rows, iqs[0].scale, iqs[0].zero_point, static_cast<float *>(c), io_.stream());
      } else {
        // one scale per row (input_per_channel_, :152-171), narrowed to float (:168-171); the zero point used is
        // the first one (matmul_dynamic_int8.cc:61)
        if (iqs.size() != static_cast<size_t>(rows)) return kLiteError;
        std::vector<mi_dq_params> ps(iqs.size());
        for (size_t i = 0; i < iqs.size(); ++i) {
          ps[i] = mi_dq_params{iqs[i].scale, static_cast<float>(iqs[i].scale), iqs[0].zero_point, 0.0f, 0.0f};
        }
        const size_t bytes = ps.size() * sizeof(mi_dq_params);
        void *dev = row_params_.Reserve(bytes);
        if (dev == nullptr || mi_copy_to_device(dev, ps.data(), bytes, io_.stream()) != MI_OK) return kLiteError;
        rc = mi_dynmm_run_rows(dyn_, a, rows, static_cast<const mi_dq_params *>(dev), static_cast<float *>(c),
                               io_.stream());
      }
    }
    return rc == MI_OK ? io_.Deliver(&outputs_[0]) : static_cast<int>(kLiteError);
  }

 private:
  static constexpr int32_t kSiblingMaxRows = 32;  // the row counts that mi_matmul_run_group runs as one launch
  static constexpr int32_t kDecodeMaxRows = 64;   // the row counts that the blocked second copy of the weights serves
                                                  // (twice as many against at most 4096 channels with K >= 1024)
  static constexpr int kNotGrouped = -1000;

  // Runs this kernel and every sibling that is ready for the same rows as one launch.  kNotGrouped: nothing was
  // launched (no sibling qualifies) and the caller goes on alone.
  int ExecuteWithSiblings(int32_t rows) {
    std::vector<MatmulKernel *> run;
    run.push_back(this);
    const bool dynamic = dyn_ != nullptr;
    for (MatmulKernel *m : group_->Members()) {
      if (m == this || (dynamic ? m->dyn_ == nullptr : m->full_ == nullptr)) continue;
      if (RowsOfOutput(m->outputs_[0]) != rows || m->inputs_[0].ElementNum() != static_cast<int64_t>(rows) * k_) continue;
      run.push_back(m);
    }
    if (run.size() < 2) return kNotGrouped;
    // a dynamic MatMul reads its input's scale and zero point at every run: where DynamicQuant left them on the
    // device, or one pair from the tensor; one pair per row on the host keeps the members apart (each uploads its own)
    QuantOnDevice on_dev;
    const bool quant_on_device = dynamic && inputs_[0].GetDeviceData() != nullptr &&
                                 Published::Quant(inputs_[0].GetDeviceData(), &on_dev) &&
                                 (!on_dev.per_row || on_dev.rows == rows);
    const auto iqs = dynamic && !quant_on_device ? inputs_[0].QuantParams() : std::vector<QuantParam>();
    if (dynamic && !quant_on_device && iqs.size() != 1) return kNotGrouped;
    const auto *a = static_cast<const int8_t *>(io_.Input(&inputs_[0]));
    if (a == nullptr) return kLiteNullptr;
    if (dynamic && quant_on_device && a != inputs_[0].GetDeviceData()) return kNotGrouped;
    std::vector<void *> outs;
    for (MatmulKernel *m : run) {
      void *c = m->io_.Output(m->outputs_[0].DataSize());
      if (c == nullptr) return kLiteNullptr;
      outs.push_back(c);
    }
    int rc = MI_ERROR;
    if (dynamic) {
      std::vector<mi_dynmm *> handles;
      for (MatmulKernel *m : run) handles.push_back(m->dyn_);
      rc = mi_dynmm_run_group(handles.data(), static_cast<int32_t>(handles.size()), a, rows,
                              quant_on_device ? 0.0 : iqs[0].scale, quant_on_device ? 0 : iqs[0].zero_point,
                              quant_on_device ? on_dev.params : nullptr, quant_on_device && on_dev.per_row ? 1 : 0,
                              reinterpret_cast<float *const *>(outs.data()), io_.stream());
    } else {
      std::vector<mi_matmul *> handles;
      for (MatmulKernel *m : run) handles.push_back(m->full_);
      rc = mi_matmul_run_group(handles.data(), static_cast<int32_t>(handles.size()), a, rows,
                               reinterpret_cast<int8_t *const *>(outs.data()), io_.stream());
    }
    if (rc != MI_OK) return kLiteError;
    g_group_launches.fetch_add(1, std::memory_order_relaxed);
    for (MatmulKernel *m : run) {
      if (m == this) continue;
      m->computed_by_sibling_ = true;
      m->sibling_rows_ = rows;
      m->sibling_host_ = inputs_[0].Data().get();
      m->sibling_dev_ = inputs_[0].GetDeviceData();
      m->sibling_version_ = Published::Version(m->sibling_dev_);
    }
    return io_.Deliver(&outputs_[0]);
  }

  // A constant weight of rank > 2: output matrix i = activation matrix a_offsets[i] x weight matrix b_offsets[i], the
  // indices by the reference's broadcast rule (MatmulBaseInt8CPUKernel::Run, matmul_base_int8.cc:549-568).
  int ExecuteBatched() {
    const auto ashape = inputs_[0].Shape(), wshape = inputs_[kWeightIndex].Shape();
    if (ashape.size() < 2 || ashape.size() > MI_MAX_DIMS || wshape.size() > MI_MAX_DIMS || ashape.back() != k_) return kLiteError;
    if (inputs_[0].ElementNum() == 0) return kSuccess;
    std::vector<int32_t> a32(ashape.begin(), ashape.end()), w32(wshape.begin(), wshape.end());
    int32_t batch = 0;
    const int64_t cap = outputs_[0].ElementNum() / n_;  // at least one row per output matrix
    std::vector<int32_t> a_off(static_cast<size_t>(cap)), b_off(static_cast<size_t>(cap));
    if (mi_matmul_broadcast_offsets(a32.data(), static_cast<int32_t>(a32.size()), w32.data(),
                                    static_cast<int32_t>(w32.size()), static_cast<int32_t>(cap), &batch, a_off.data(),
                                    b_off.data()) != MI_OK) {
      return kLiteError;
    }
    const int32_t rows = static_cast<int32_t>(ashape[ashape.size() - 2]);
    if (outputs_[0].ElementNum() != static_cast<int64_t>(batch) * rows * n_) return kLiteError;
    const auto *a = static_cast<const int8_t *>(io_.Input(&inputs_[0]));
    void *c = io_.Output(outputs_[0].DataSize());
    if (a == nullptr || c == nullptr) return kLiteNullptr;
    if (mi_matmul_run_batched(full_, a, rows, batch, a_off.data(), b_off.data(), static_cast<int8_t *>(c),
                              io_.stream()) != MI_OK) {
      return kLiteError;
    }
    return io_.Deliver(&outputs_[0]);
  }

  bool b_transpose_;
  int act_;
  int32_t k_ = 0, n_ = 0;
  bool batched_ = false;
  std::shared_ptr<SiblingGroup> group_;
  bool computed_by_sibling_ = false;  // the output buffer already holds this run's result
  int32_t sibling_rows_ = 0;          // ... for this row count and this input memory
  const void *sibling_host_ = nullptr;
  void *sibling_dev_ = nullptr;
  int64_t sibling_version_ = 0;
  mi_matmul *full_ = nullptr;
  mi_dynmm *dyn_ = nullptr;
  DeviceIo io_;
  DeviceBuffer row_params_;
};

std::shared_ptr<kernel::Kernel> MatmulCreator(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out,
                                              const schema::Primitive *prim, const Context *ctx) {
  if (!LibraryReady() || in.size() < 2 || out.size() != 1 || prim == nullptr) return nullptr;
  bool b_transpose = true;
  int act = 0;
  if (const auto *fc = prim->value_as_FullConnection()) {  // weight is always [N, K] (fullconnection_int8.cc:33-34)
    // use_axis only changes how the input's dimensions fold into rows x K, which the kernel takes from the output
    // shape and the weight exactly as the reference does (fullconnection_int8.cc:49-58)
    act = fc->activation_type();
  } else if (const auto *mm = prim->value_as_MatMulFusion()) {
    if (mm->transpose_a()) return nullptr;
    b_transpose = mm->transpose_b();
    act = mm->activation_type();
  } else {
    return nullptr;
  }
  const MSTensor &w = in[kWeightIndex];
  const bool out_i8 = out[0].DataType() == DataType::kNumberTypeInt8;
  const bool out_f32 = out[0].DataType() == DataType::kNumberTypeFloat32;
  if (!w.IsConst() || w.DataType() != DataType::kNumberTypeInt8 || w.Shape().size() < 2) return nullptr;
  // a weight of rank > 2 (a batch of matrices) is taken for the full-quant MatMul; FullConnection has none, and the
  // dynamic MatMul's batched form stays with the builtin kernel
  const bool batched_w = w.Shape().size() > 2;
  if (batched_w && (prim->value_as_MatMulFusion() == nullptr || !out_i8 || w.Shape().size() > MI_MAX_DIMS)) return nullptr;
  // full quant needs per-tensor activations; the dynamic MatMul also takes one input scale per row
  if (!(out_i8 || out_f32) || (out_i8 && (!PerTensor(in[0]) || !PerTensor(out[0])))) return nullptr;
  if (act != MI_ACT_NONE && act != MI_ACT_RELU && act != MI_ACT_RELU6) return nullptr;
  if (in.size() > kBiasIndex) {
    const auto want = out_i8 ? DataType::kNumberTypeInt32 : DataType::kNumberTypeFloat32;
    if (!in[kBiasIndex].IsConst() || in[kBiasIndex].DataType() != want) return nullptr;
  }
  // everything Prepare / Execute would otherwise fail on is screened here, where declining still lets the scheduler
  // fall back: the activation type, quant parameters present and of a usable count, the contraction length
  // (a dynamic-quant MatMul finds its input's scale on the tensor only at run time: DynamicQuant writes it there)
  if (in[0].DataType() != DataType::kNumberTypeInt8) return nullptr;
  const auto wshape = w.Shape();
  const size_t wr = wshape.size();
  const int64_t n = b_transpose ? wshape[wr - 2] : wshape[wr - 1], k = b_transpose ? wshape[wr - 1] : wshape[wr - 2];
  for (size_t i = 0; i + 2 < wr; ++i)
    if (wshape[i] <= 0) return nullptr;
  const size_t nfilter = w.QuantParams().size();
  if (n <= 0 || k <= 0 || (nfilter != 1 && nfilter != static_cast<size_t>(n))) return nullptr;
  const auto ashape = in[0].Shape();
  bool known = !ashape.empty();
  int64_t elements = 1;
  for (int64_t d : ashape) {
    known = known && d >= 0;
    elements *= d;
  }
  if (known) {
    if (prim->value_as_MatMulFusion() != nullptr ? ashape.back() != k : elements % k != 0) return nullptr;
    if (batched_w) {  // the batch extents must broadcast (InitBroadcastParams, matmul_fp32_base.cc:611-620)
      if (ashape.size() < 2 || ashape.size() > MI_MAX_DIMS) return nullptr;
      std::vector<int32_t> a32(ashape.begin(), ashape.end()), w32(wshape.begin(), wshape.end());
      int32_t batch = 0;
      std::vector<int32_t> ao(1 << 16), bo(1 << 16);
      if (mi_matmul_broadcast_offsets(a32.data(), static_cast<int32_t>(a32.size()), w32.data(),
                                      static_cast<int32_t>(w32.size()), 1 << 16, &batch, ao.data(), bo.data()) != MI_OK) {
        return nullptr;
      }
    }
  }
  return std::make_shared<MatmulKernel>(in, out, prim, ctx, b_transpose, act);
}

// ---- Conv2DFusion int8 -------------------------------------------------------------------------------------------
class ConvKernel : public kernel::Kernel {
 public:
  using Kernel::Kernel;
  ~ConvKernel() override {
    io_.Withdraw(&outputs_[0]);
    mi_conv_destroy(conv_);
  }

  int Prepare() override {
    io_.Configure(context_, GetConfig("mi355x"), outputs_[0].Name());
    return Build();
  }

  // Weights and quant parameters do not depend on the image size; SAME-mode padding does (the builtin kernel gets
  // it from shape inference at every resize, conv2d_infer.c:34-50), so the handle is rebuilt only when it moved.
  int ReSize() override {
    if (conv_ == nullptr) return kSuccess;  // Prepare has not run yet
    mi_conv_desc d{};
    FillGeometry(&d);
    if (d.pad_u == pads_[0] && d.pad_d == pads_[1] && d.pad_l == pads_[2] && d.pad_r == pads_[3]) return kSuccess;
    mi_conv_destroy(conv_);
    conv_ = nullptr;
    return Build();
  }

  int Execute() override {
    const auto s = inputs_[0].Shape();
    if (s.size() != 4) return kLiteError;
    if (inputs_[0].ElementNum() == 0 || outputs_[0].ElementNum() == 0) return kSuccess;
    const auto *x = static_cast<const int8_t *>(io_.Input(&inputs_[0]));
    auto *y = static_cast<int8_t *>(io_.Output(outputs_[0].DataSize()));
    if (x == nullptr || y == nullptr) return kLiteNullptr;
    if (mi_conv_run(conv_, x, static_cast<int32_t>(s[0]), static_cast<int32_t>(s[1]), static_cast<int32_t>(s[2]), y,
                    io_.stream()) != MI_OK) {
      return kLiteError;
    }
    return io_.Deliver(&outputs_[0]);
  }

 private:
  void FillGeometry(mi_conv_desc *d) const {
    const auto *cv = primitive_->value_as_Conv2DFusion();
    const auto in_shape = inputs_[0].Shape();  // NHWC
    d->in_channel = static_cast<int32_t>(cv->in_channel());
    d->out_channel = static_cast<int32_t>(cv->out_channel());
    d->kernel_h = static_cast<int32_t>(cv->kernel_size()->Get(0));
    d->kernel_w = static_cast<int32_t>(cv->kernel_size()->Get(1));
    d->stride_h = static_cast<int32_t>(cv->stride()->Get(0));
    d->stride_w = static_cast<int32_t>(cv->stride()->Get(1));
    d->dilation_h = static_cast<int32_t>(cv->dilation()->Get(0));
    d->dilation_w = static_cast<int32_t>(cv->dilation()->Get(1));
    d->group = static_cast<int32_t>(cv->group());
    d->act_type = cv->activation_type();
    if (cv->pad_mode() == schema::PadMode_SAME && in_shape.size() == 4) {
      int32_t oh = 0, ow = 0;
      mi_conv_same_pad(static_cast<int32_t>(in_shape[1]), d->kernel_h, d->stride_h, d->dilation_h, &d->pad_u,
                       &d->pad_d, &oh);
      mi_conv_same_pad(static_cast<int32_t>(in_shape[2]), d->kernel_w, d->stride_w, d->dilation_w, &d->pad_l,
                       &d->pad_r, &ow);
    } else if (cv->pad_mode() == schema::PadMode_PAD && cv->pad_list() != nullptr && cv->pad_list()->size() == 4) {
      d->pad_u = static_cast<int32_t>(cv->pad_list()->Get(0));
      d->pad_d = static_cast<int32_t>(cv->pad_list()->Get(1));
      d->pad_l = static_cast<int32_t>(cv->pad_list()->Get(2));
      d->pad_r = static_cast<int32_t>(cv->pad_list()->Get(3));
    }
  }

  int Build() {
    const MSTensor &w = inputs_[kWeightIndex];
    mi_conv_desc d{};
    FillGeometry(&d);
    pads_[0] = d.pad_u, pads_[1] = d.pad_d, pads_[2] = d.pad_l, pads_[3] = d.pad_r;
    const auto iq = inputs_[0].QuantParams().front();
    const auto oq = outputs_[0].QuantParams().front();
    d.in_scale = iq.scale;
    d.in_zp = iq.zero_point;
    d.out_scale = oq.scale;
    d.out_zp = oq.zero_point;
    std::vector<double> scales;
    std::vector<int32_t> zps;
    FilterQuant(w, &scales, &zps);
    d.filter_quant_num = static_cast<int32_t>(scales.size());
    d.filter_scales = scales.data();
    d.filter_zps = zps.data();
    d.flags = Exact3x3() ? MI_CONV_3X3_EXACT : 0;
    const void *bias = inputs_.size() > kBiasIndex ? inputs_[kBiasIndex].Data().get() : nullptr;
    // MI_NOT_SUPPORT (3x3 stride-1 Winograd case, grouped convolution) surfaces here as an error; the creator
    // below screens those cases out first so that the scheduler falls back instead
    return ToStatus(
      mi_conv_create(&d, static_cast<const int8_t *>(w.Data().get()), static_cast<const int32_t *>(bias), &conv_));
  }

  int32_t pads_[4] = {0, 0, 0, 0};
  mi_conv *conv_ = nullptr;
  DeviceIo io_;
};

std::shared_ptr<kernel::Kernel> ConvCreator(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out,
                                            const schema::Primitive *prim, const Context *ctx) {
  if (!LibraryReady() || in.size() < 2 || out.size() != 1 || prim == nullptr) return nullptr;
  const auto *cv = prim->value_as_Conv2DFusion();
  if (cv == nullptr || cv->kernel_size() == nullptr || cv->stride() == nullptr || cv->dilation() == nullptr) {
    return nullptr;
  }
  const MSTensor &w = in[kWeightIndex];
  if (!w.IsConst() || w.DataType() != DataType::kNumberTypeInt8 || out[0].DataType() != DataType::kNumberTypeInt8) {
    return nullptr;
  }
  if (in[0].DataType() != DataType::kNumberTypeInt8 || !PerTensor(in[0]) || !PerTensor(out[0])) return nullptr;
  if (in.size() > kBiasIndex &&
      (!in[kBiasIndex].IsConst() || in[kBiasIndex].DataType() != DataType::kNumberTypeInt32)) {
    return nullptr;
  }
  const size_t nfilter = w.QuantParams().size();  // per tensor or one per output channel (convolution_base.cc:377-397)
  if (cv->out_channel() <= 0 || (nfilter != 1 && nfilter != static_cast<size_t>(cv->out_channel()))) return nullptr;
  const int64_t kh = cv->kernel_size()->Get(0), kw = cv->kernel_size()->Get(1);
  const bool depthwise = cv->group() > 1 && cv->group() == cv->in_channel() && cv->group() == cv->out_channel();
  if (cv->group() != 1 && !depthwise) return nullptr;
  // on x86 the reference runs its integer Winograd for dense 3x3 stride-1 dilation-1 convolutions
  // (convolution_int8_creator.cc:81-94), whose results are not those of the exact convolution: leave them to it
  // unless the deployment asked for the exact convolution (the reference's choice on ARM64 with dot product)
  if (!depthwise && kh == 3 && kw == 3 && cv->stride()->Get(0) == 1 && cv->stride()->Get(1) == 1 &&
      cv->dilation()->Get(0) == 1 && cv->dilation()->Get(1) == 1 && !Exact3x3()) {
    return nullptr;
  }
  return std::make_shared<ConvKernel>(in, out, prim, ctx);
}

// ---- DynamicQuant, fp32 -> int8 per tensor -------------------------------------------------------------------------
class DynamicQuantKernel : public kernel::Kernel {
 public:
  using Kernel::Kernel;
  ~DynamicQuantKernel() override {
    io_.Withdraw(&outputs_[0]);
    mi_dynquant_destroy(dq_);
  }

  int Prepare() override {
    io_.Configure(context_, GetConfig("mi355x"), outputs_[0].Name());
    const auto *p = primitive_->value_as_DynamicQuant();
    per_row_ = p->prefer_axes() != nullptr && p->prefer_axes()->size() > 0;
    return ToStatus(mi_dynquant_create(p->symmetric() ? 1 : 0, &dq_));
  }
  int ReSize() override { return kSuccess; }
  int Execute() override {
    const int64_t n = inputs_[0].ElementNum();
    if (n == 0) return kSuccess;
    const auto *x = static_cast<const float *>(io_.Input(&inputs_[0]));
    auto *q = static_cast<int8_t *>(io_.Output(outputs_[0].DataSize()));
    if (x == nullptr || q == nullptr) return kLiteNullptr;
    // The scales and zero points stay on the device for the consumers of this provider (QuantOnDevice).  A builtin
    // consumer reads them from the tensor, so they also travel to the host -- as a copy into page-locked memory
    // queued behind the kernels, complete once Deliver has waited for the output's own copy: one wait per run instead
    // of two.  An output declared device-only has no builtin consumer: nothing is waited for, and the tensor's quant
    // parameters are left as they are.
    QuantOnDevice quant;
    quant.per_row = per_row_;
    size_t blocks = 1;
    if (per_row_) {  // the creator admitted only "every axis but the last": one run per row of the last axis
      const int64_t unit = inputs_[0].Shape().back();
      const int64_t segments = n / unit;
      blocks = static_cast<size_t>(segments);
      auto *dev = static_cast<mi_dq_params *>(row_params_.Reserve(blocks * sizeof(mi_dq_params)));
      if (dev == nullptr || mi_dynquant_run_segments(dq_, x, segments, unit, q, dev, io_.stream()) != MI_OK) {
        return kLiteError;
      }
      quant.params = dev;
      quant.rows = segments;
    } else {
      if (mi_dynquant_run(dq_, x, n, q, io_.stream()) != MI_OK) return kLiteError;
      quant.params = mi_dynquant_device_params(dq_);
    }
    if (!io_.host_copy()) return io_.Deliver(&outputs_[0], &quant);
    const size_t bytes = blocks * sizeof(mi_dq_params);
    auto *ps = static_cast<mi_dq_params *>(host_params_.Reserve(bytes));
    if (ps == nullptr || mi_copy_to_host_async(ps, quant.params, bytes, io_.stream()) != MI_OK) return kLiteError;
    const int rc = io_.Deliver(&outputs_[0], &quant);  // copies the output to the host and waits for the stream
    if (rc != kSuccess) return rc;
    // what DynamicQuantCPUKernel::CalculatePerlayerScaleZp / CalculatePerChannelScaleZp publish on the output tensor
    // (dynamic_quant.cc:156-218)
    std::vector<QuantParam> qps(blocks);
    for (size_t i = 0; i < blocks; ++i) {
      qps[i].bit_num = 8;
      qps[i].scale = ps[i].scale;
      qps[i].zero_point = ps[i].zero_point;
      qps[i].min = ps[i].real_min;
      qps[i].max = ps[i].real_max;
    }
    outputs_[0].SetQuantParams(qps);
    return kSuccess;
  }

 private:
  // page-locked host memory (grows, never shrinks)
  class PinnedBuffer {
   public:
    PinnedBuffer() = default;
    PinnedBuffer(const PinnedBuffer &) = delete;
    PinnedBuffer &operator=(const PinnedBuffer &) = delete;
    ~PinnedBuffer() { mi_host_free(p_); }
    void *Reserve(size_t bytes) {
      if (bytes > cap_) {
        mi_host_free(p_);
        p_ = nullptr;
        cap_ = 0;
        if (mi_host_malloc(bytes, &p_) != MI_OK) return nullptr;
        cap_ = bytes;
      }
      return p_;
    }

   private:
    void *p_ = nullptr;
    size_t cap_ = 0;
  };

  mi_dynquant *dq_ = nullptr;
  bool per_row_ = false;
  DeviceIo io_;
  DeviceBuffer row_params_;
  PinnedBuffer host_params_;
};

std::shared_ptr<kernel::Kernel> DynamicQuantCreator(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out,
                                                    const schema::Primitive *prim, const Context *ctx) {
  if (!LibraryReady() || in.size() != 1 || out.size() != 1 || prim == nullptr) return nullptr;
  const auto *p = prim->value_as_DynamicQuant();
  if (p == nullptr) return nullptr;
  if (p->prefer_axes() != nullptr && p->prefer_axes()->size() > 0) {
    // per-channel activation scales: taken when the preferred axes are exactly the leading rank-1 axes (what the
    // converter emits for a MatMul input without transpose_a, insert_quant_node_manager.cc:138-160), so that no
    // transposition is involved; everything else stays with the builtin kernel
    const size_t rank = in[0].Shape().size();
    if (rank < 2 || p->prefer_axes()->size() != rank - 1) return nullptr;
    for (size_t i = 0; i + 1 < rank; ++i) {
      const int axis = p->prefer_axes()->Get(i);
      if ((axis < 0 ? axis + static_cast<int>(rank) : axis) != static_cast<int>(i)) return nullptr;
    }
  }
  if (p->dst_type() != static_cast<int64_t>(DataType::kNumberTypeInt8)) return nullptr;
  if (in[0].DataType() != DataType::kNumberTypeFloat32 || out[0].DataType() != DataType::kNumberTypeInt8) {
    return nullptr;
  }
  return std::make_shared<DynamicQuantKernel>(in, out, prim, ctx);
}

// ---- registration: arch "CPU" for applications, arch "" for the stock benchmark tool --------------------------------
namespace {
struct Registrar {
  Registrar() {
    for (const char *arch : {"CPU", ""}) {
      registry::RegisterKernel::RegKernel(arch, "mi355x", DataType::kNumberTypeInt8, schema::PrimitiveType_MatMulFusion,
                                          MatmulCreator);
      registry::RegisterKernel::RegKernel(arch, "mi355x", DataType::kNumberTypeInt8,
                                          schema::PrimitiveType_FullConnection, MatmulCreator);
      registry::RegisterKernel::RegKernel(arch, "mi355x", DataType::kNumberTypeInt8, schema::PrimitiveType_Conv2DFusion,
                                          ConvCreator);
      registry::RegisterKernel::RegKernel(arch, "mi355x", DataType::kNumberTypeFloat32,
                                          schema::PrimitiveType_DynamicQuant, DynamicQuantCreator);
    }
  }
} g_registrar;
}  // namespace

// How many times sibling MatMuls went out as one launch (for tests and for checking that a model's siblings were found).
extern "C" int64_t mi355x_provider_group_launches() { return g_group_launches.load(std::memory_order_relaxed); }
// How many sessions currently hold a stream (for tests: destroying a session's last kernel gives its stream back).
extern "C" int64_t mi355x_provider_session_streams() { return static_cast<int64_t>(SessionStreams::Count()); }
}  // namespace mi355x
}  // namespace mindspore
