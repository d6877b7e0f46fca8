// TEST INFRASTRUCTURE.  Plays the part of the Lite scheduler for mindspore_amd/provider/mi355x_provider.cc, compiled
// against the stand-in API of this directory: infers the node's shape (through a provider's KernelInterface when one
// is registered for the operator, else through the stand-in for the builtin inference below -- and, as
// Scheduler::InferNodeShape does, only the builtin path leaves the node an OpParameter, scheduler.cc:652-698), looks
// the creator up by (arch, provider, data type, op type) as scheduler.cc:1131-1177 does, runs Prepare / ReSize /
// Execute, and hands tensors in and out through a C interface for the Python tests.  The provider source is
// included, so its static registrar runs when this library is loaded.
#include <string.h>

#include <map>
#include <memory>
#include <string>
#include <vector>

#include <thread>

#include "../../mindspore_amd/provider/mi355x_allocator.h"
#include "../../mindspore_amd/provider/mi355x_provider.cc"
#include "include/kernel_interface.h"
#include "include/registry/register_kernel_interface.h"

using mindspore::MSTensor;
namespace schema = mindspore::schema;

extern "C" {
typedef struct ph_tensor {
  int32_t dtype;  // mindspore::DataType id
  int32_t dims;
  int64_t shape[8];
  const void *data;  // NULL: not materialised (an activation before the first run)
  int64_t bytes;
  int32_t is_const;
  int32_t nquant;
  const double *scales;
  const int32_t *zps;
} ph_tensor;

typedef struct ph_op {
  int32_t type;  // schema::PrimitiveType id
  int32_t transpose_a, transpose_b, act;
  int32_t has_bias, use_axis, axis;
  int64_t kernel[2], stride[2], dilation[2], pad_list[4];
  int32_t has_pad_list, pad_mode;
  int64_t group, in_channel, out_channel;
  int32_t symmetric;
  int64_t dst_type;
  int32_t n_prefer_axes;
  int32_t prefer_axes[8];
} ph_op;
}

namespace {
// kDeclined: the creator returned nullptr and the node has an OpParameter, i.e. the scheduler now takes the builtin CPU
// kernel.  kDeclinedNoFallback: it returned nullptr after a provider's KernelInterface had inferred the node, so that
// there is no OpParameter and FindBackendKernel gives up (scheduler.cc:1178-1183): Model::Build fails.
enum Stage { kOk = 0, kNoCreator = 1, kDeclined = 2, kInferFailed = 3, kPrepareFailed = 4, kResizeFailed = 5, kExecuteFailed = 6,
             kDeclinedNoFallback = 7 };

// Stand-in for the builtin (nnacl) shape inference of the four operator types: output shapes from the library's
// mi_infer_* functions, which tests/test_infer_shape.py checks against the compiled nnacl functions.
class BuiltinInference : public mindspore::kernel::KernelInterface {
 public:
  mindspore::Status Infer(std::vector<MSTensor> *inputs, std::vector<MSTensor> *outputs,
               const schema::Primitive *primitive) override {
    if (inputs == nullptr || outputs == nullptr || primitive == nullptr || inputs->empty() || outputs->size() != 1) {
      return mindspore::kLiteInferError;
    }
    const auto dims = [](const MSTensor &t) {
      std::vector<int32_t> v;
      for (int64_t d : t.Shape()) v.push_back(static_cast<int32_t>(d));
      return v;
    };
    int32_t out[MI_MAX_DIMS] = {0};
    int32_t out_dims = 0;
    int ret = MI_INFER_ERR;
    const size_t n = inputs->size();
    const std::vector<int32_t> a = dims((*inputs)[0]);
    const std::vector<int32_t> b = n > 1 ? dims((*inputs)[1]) : std::vector<int32_t>();
    const std::vector<int32_t> bias = n > 2 ? dims((*inputs)[2]) : std::vector<int32_t>();
    if (a.size() > MI_MAX_DIMS || b.size() > MI_MAX_DIMS || bias.size() > MI_MAX_DIMS) return mindspore::kLiteInferError;
    switch (primitive->value_type()) {
      case schema::PrimitiveType_MatMulFusion: {
        const auto *mm = primitive->value_as_MatMulFusion();
        if (mm == nullptr || (n != 2 && n != 3)) return mindspore::kLiteInferError;
        ret = mi_infer_matmul(a.data(), static_cast<int32_t>(a.size()), b.data(), static_cast<int32_t>(b.size()),
                              bias.data(), static_cast<int32_t>(bias.size()), mm->transpose_a(), mm->transpose_b(), out,
                              &out_dims);
        break;
      }
      case schema::PrimitiveType_FullConnection: {
        const auto *fc = primitive->value_as_FullConnection();
        if (fc == nullptr || n < 2) return mindspore::kLiteInferError;
        ret = mi_infer_fullconnection(a.data(), static_cast<int32_t>(a.size()), b.data(),
                                      static_cast<int32_t>(b.size()), bias.data(), static_cast<int32_t>(bias.size()),
                                      fc->has_bias(), fc->use_axis(), static_cast<int32_t>(fc->axis()), out, &out_dims);
        break;
      }
      case schema::PrimitiveType_Conv2DFusion: {
        const auto *cv = primitive->value_as_Conv2DFusion();
        if (cv == nullptr || (n != 2 && n != 3)) return mindspore::kLiteInferError;
        // attribute defaults as the builtin populate step fills them (ops/populate/conv2d_populate.cc)
        mi_conv_infer p{};
        const auto at = [](const flatbuffers::Vector<int64_t> *v, uint32_t i, int32_t dflt) {
          return v != nullptr && v->size() > i ? static_cast<int32_t>(v->Get(i)) : dflt;
        };
        p.kernel_h = at(cv->kernel_size(), 0, -1);
        p.kernel_w = at(cv->kernel_size(), 1, -1);
        p.stride_h = at(cv->stride(), 0, 1);
        p.stride_w = at(cv->stride(), 1, 1);
        p.dilation_h = at(cv->dilation(), 0, 1);
        p.dilation_w = at(cv->dilation(), 1, 1);
        p.pad_mode = cv->pad_mode() == schema::PadMode_SAME    ? MI_PAD_SAME
                     : cv->pad_mode() == schema::PadMode_VALID ? MI_PAD_VALID
                                                               : MI_PAD_EXPLICIT;
        const bool has_pads = cv->pad_list() != nullptr && cv->pad_list()->size() >= 4;
        p.pad_u = has_pads ? at(cv->pad_list(), 0, 0) : 0;
        p.pad_d = has_pads ? at(cv->pad_list(), 1, 0) : 0;
        p.pad_l = has_pads ? at(cv->pad_list(), 2, 0) : 0;
        p.pad_r = has_pads ? at(cv->pad_list(), 3, 0) : 0;
        p.group = static_cast<int32_t>(cv->group());
        ret = mi_infer_conv2d(a.data(), static_cast<int32_t>(a.size()), b.data(), static_cast<int32_t>(b.size()), &p,
                              out, &out_dims);
        break;
      }
      case schema::PrimitiveType_DynamicQuant: {  // same shape as the input (dynamic_quant_infer.c:21-40)
        for (int32_t d : a) {
          if (d < 0) return mindspore::kLiteInferInvalid;
        }
        (*outputs)[0].SetFormat((*inputs)[0].format());
        (*outputs)[0].SetShape((*inputs)[0].Shape());
        return mindspore::kSuccess;
      }
      default:
        return mindspore::kLiteInferError;
    }
    (*outputs)[0].SetFormat((*inputs)[0].format());
    if (ret == MI_INFER_INVALID) return mindspore::kLiteInferInvalid;
    if (ret != MI_OK) return mindspore::kLiteInferError;
    (*outputs)[0].SetShape(std::vector<int64_t>(out, out + out_dims));
    return mindspore::kSuccess;
  }
};




struct Session {
  schema::Primitive prim;
  std::vector<MSTensor> inputs, outputs;
  std::shared_ptr<mindspore::kernel::Kernel> kernel;
  std::shared_ptr<mindspore::kernel::KernelInterface> infer;  // a provider's, or nullptr: builtin inference
  bool has_op_parameter = false;
  mindspore::Context ctx;
  const mindspore::Context *session_ctx = &ctx;  // nodes linked to a producer belong to the producer's session
  std::map<std::string, std::map<std::string, std::string>> config;  // the session's config file sections
};

std::vector<mindspore::QuantParam> Quant(int n, const double *scales, const int32_t *zps) {
  std::vector<mindspore::QuantParam> q;
  for (int i = 0; i < n; ++i) q.push_back({8, scales[i], zps[i], 0.0, 0.0});
  return q;
}

MSTensor Tensor(const ph_tensor &t, const std::string &name) {
  MSTensor ms(name, static_cast<mindspore::DataType>(t.dtype), std::vector<int64_t>(t.shape, t.shape + t.dims), t.data,
              static_cast<size_t>(t.bytes), t.is_const != 0);
  ms.SetQuantParams(Quant(t.nquant, t.scales, t.zps));
  return ms;
}

void Fill(const ph_op &op, schema::Primitive *p) {
  p->type_ = static_cast<schema::PrimitiveType>(op.type);
  const auto act = static_cast<schema::ActivationType>(op.act);
  p->matmul_.transpose_a_ = op.transpose_a != 0;
  p->matmul_.transpose_b_ = op.transpose_b != 0;
  p->matmul_.activation_type_ = act;
  p->fc_.has_bias_ = op.has_bias != 0;
  p->fc_.use_axis_ = op.use_axis != 0;
  p->fc_.axis_ = op.axis;
  p->fc_.activation_type_ = act;
  p->conv_.kernel_size_ = flatbuffers::Vector<int64_t>({op.kernel[0], op.kernel[1]});
  p->conv_.stride_ = flatbuffers::Vector<int64_t>({op.stride[0], op.stride[1]});
  p->conv_.dilation_ = flatbuffers::Vector<int64_t>({op.dilation[0], op.dilation[1]});
  p->conv_.pad_list_ = flatbuffers::Vector<int64_t>({op.pad_list[0], op.pad_list[1], op.pad_list[2], op.pad_list[3]});
  p->conv_.has_pad_list_ = op.has_pad_list != 0;
  p->conv_.pad_mode_ = static_cast<schema::PadMode>(op.pad_mode);
  p->conv_.group_ = op.group;
  p->conv_.in_channel_ = op.in_channel;
  p->conv_.out_channel_ = op.out_channel;
  p->conv_.activation_type_ = act;
  p->dynquant_.symmetric_ = op.symmetric != 0;
  p->dynquant_.dst_type_ = op.dst_type;
  p->dynquant_.has_prefer_axes_ = op.n_prefer_axes > 0;
  p->dynquant_.prefer_axes_ = flatbuffers::Vector<int32_t>(std::vector<int32_t>(op.prefer_axes, op.prefer_axes + op.n_prefer_axes));
}

int Infer(Session *s) {
  if (s->infer != nullptr) {  // a provider answered: InferNodeShape returns before it makes the OpParameter
    s->has_op_parameter = false;
    return s->infer->Infer(&s->inputs, &s->outputs, &s->prim).IsOk() ? kOk : kInferFailed;
  }
  s->has_op_parameter = true;
  BuiltinInference builtin;
  return builtin.Infer(&s->inputs, &s->outputs, &s->prim).IsOk() ? kOk : kInferFailed;
}

// A KernelInterface that a test may register under the provider name to see what registering one for a builtin
// operator does to the fallback (the provider itself registers none).
std::shared_ptr<mindspore::kernel::KernelInterface> TestInterfaceCreator() { return std::make_shared<BuiltinInference>(); }
}  // namespace

extern "C" {
// Builds the node: tensors, shape inference, creator lookup and call, Prepare().  *stage tells how far it got;
// *code is the status of the failing call (0 otherwise).  Returns NULL unless the kernel is ready to execute.
// `producer` (optional): a node made earlier whose output tensor becomes this node's input 0 -- the same tensor
// object, as in a graph, so that what the producer leaves on it (data, quant params, device address) is what this
// node finds.  `out_name` names the output tensor; `device_only_outputs` (optional) is the value of that key in the
// [mi355x] section of the session config.
void *ph_create_node(const ph_op *op, const char *arch, const char *provider, const ph_tensor *inputs, int32_t n_in,
                     int32_t out_dtype, int32_t out_nquant, const double *out_scales, const int32_t *out_zps,
                     void *producer, const char *out_name, const char *device_only_outputs, int32_t *stage,
                     int32_t *code) {
  auto s = std::make_unique<Session>();
  *stage = kOk;
  *code = 0;
  Fill(*op, &s->prim);
  if (device_only_outputs != nullptr) s->config["mi355x"]["device_only_outputs"] = device_only_outputs;
  for (int i = 0; i < n_in; ++i) {
    if (i == 0 && producer != nullptr) {
      s->inputs.push_back(static_cast<Session *>(producer)->outputs[0]);
      s->session_ctx = static_cast<Session *>(producer)->session_ctx;
    } else {
      s->inputs.push_back(Tensor(inputs[i], "in" + std::to_string(i)));
    }
  }
  MSTensor out(out_name != nullptr ? out_name : "out", static_cast<mindspore::DataType>(out_dtype), {}, nullptr, 0,
               false);
  out.SetQuantParams(Quant(out_nquant, out_scales, out_zps));
  s->outputs.push_back(out);
  s->infer = mindspore::registry::RegisterKernelInterface::GetKernelInterface(provider, &s->prim);
  if ((*stage = Infer(s.get())) != kOk) return nullptr;
  mindspore::registry::KernelDesc desc{s->inputs[0].DataType(), op->type, arch, provider};
  auto creator = mindspore::registry::RegisterKernel::GetCreator(&s->prim, &desc);
  if (creator == nullptr) {
    *stage = kNoCreator;
    return nullptr;
  }
  s->kernel = creator(s->inputs, s->outputs, &s->prim, s->session_ctx);
  if (s->kernel == nullptr) {
    *stage = s->has_op_parameter ? kDeclined : kDeclinedNoFallback;
    return nullptr;
  }
  s->kernel->SetConfig(&s->config);  // scheduler.cc:1455-1457
  if ((*code = s->kernel->Prepare()) != 0) {
    *stage = kPrepareFailed;
    return nullptr;
  }
  return s.release();
}

void *ph_create(const ph_op *op, const char *arch, const char *provider, const ph_tensor *inputs, int32_t n_in,
                int32_t out_dtype, int32_t out_nquant, const double *out_scales, const int32_t *out_zps,
                int32_t *stage, int32_t *code) {
  return ph_create_node(op, arch, provider, inputs, n_in, out_dtype, out_nquant, out_scales, out_zps, nullptr, nullptr,
                        nullptr, stage, code);
}

// Executes a node whose input 0 is its producer's output tensor, as that producer left it.  The shape is taken from
// that tensor; when it differs from the last run the output shape is inferred again and ReSize() is called.
int32_t ph_execute_linked(void *h, int32_t *code) {
  auto *s = static_cast<Session *>(h);
  *code = 0;
  const std::vector<int64_t> before = s->outputs[0].Shape();
  if (Infer(s) != kOk) return kInferFailed;
  if (before != s->outputs[0].Shape() && (*code = s->kernel->ReSize()) != 0) return kResizeFailed;
  if ((*code = s->kernel->Execute()) != 0) return kExecuteFailed;
  return kOk;
}

// Context::SetEnableParallel of the node's own session object; nodes created later with this node as their producer
// see it in their Prepare.
void ph_set_enable_parallel(void *h, int32_t on) { static_cast<Session *>(h)->ctx.SetEnableParallel(on != 0); }

// What Model::Resize does for a node before anything is executed: infer the output shape from the producer's tensor and
// call ReSize() when it changed.
int32_t ph_resize_linked(void *h, int32_t *code) {
  auto *s = static_cast<Session *>(h);
  *code = 0;
  const std::vector<int64_t> before = s->outputs[0].Shape();
  if (Infer(s) != kOk) return kInferFailed;
  if (before != s->outputs[0].Shape() && (*code = s->kernel->ReSize()) != 0) return kResizeFailed;
  return kOk;
}

// Attaches an address to input 0 as an application could with MSTensor::SetDeviceData.
void ph_set_input_device_data(void *h, void *address) { static_cast<Session *>(h)->inputs[0].SetDeviceData(address); }

// bit 0: the output tensor has host memory; bit 1: it carries a device address.
int32_t ph_output_state(void *h) {
  auto *s = static_cast<Session *>(h);
  return (s->outputs[0].HasHostData() ? 1 : 0) | (s->outputs[0].GetDeviceData() != nullptr ? 2 : 0);
}

// Sets input 0 (new shape allowed: the output shape is inferred again and ReSize() is called, as the runtime does on
// Model::Resize), optionally its quant params (the dynamic MatMul reads them at every Execute), and executes.
int32_t ph_execute(void *h, const void *in0, const int64_t *shape, int32_t dims, int32_t nquant, const double *scales,
                   const int32_t *zps, int32_t *code) {
  auto *s = static_cast<Session *>(h);
  *code = 0;
  MSTensor &x = s->inputs[0];
  const std::vector<int64_t> new_shape(shape, shape + dims);
  const bool resized = new_shape != x.Shape();
  x.SetShape(new_shape);
  memcpy(x.MutableData(), in0, x.DataSize());
  if (nquant > 0) x.SetQuantParams(Quant(nquant, scales, zps));
  if (resized) {
    if (Infer(s) != kOk) return kInferFailed;
    if ((*code = s->kernel->ReSize()) != 0) return kResizeFailed;
  }
  if ((*code = s->kernel->Execute()) != 0) return kExecuteFailed;
  return kOk;
}

// Output tensor as the kernel left it.  Returns the number of data bytes (copied when they fit `cap`).
int64_t ph_output(void *h, int64_t *shape, int32_t *dims, void *buf, int64_t cap, double *scales, int32_t *zps,
                  int32_t max_quant, int32_t *nquant) {
  auto *s = static_cast<Session *>(h);
  MSTensor &y = s->outputs[0];
  *dims = static_cast<int32_t>(y.Shape().size());
  for (int i = 0; i < *dims && i < 8; ++i) shape[i] = y.Shape()[i];
  const auto q = y.QuantParams();
  *nquant = static_cast<int32_t>(q.size());
  for (int i = 0; i < *nquant && i < max_quant; ++i) {
    scales[i] = q[i].scale;
    zps[i] = q[i].zero_point;
  }
  const int64_t bytes = static_cast<int64_t>(y.DataSize());
  auto data = y.Data();
  if (data != nullptr && bytes <= cap) memcpy(buf, data.get(), static_cast<size_t>(bytes));
  return bytes;
}

// Shape inference alone (no GPU needed): output dims, or -1 on failure, -2 while a dimension is unknown.
int32_t ph_infer(const ph_op *op, const char *provider, const ph_tensor *inputs, int32_t n_in, int64_t *shape) {
  Session s;
  Fill(*op, &s.prim);
  for (int i = 0; i < n_in; ++i) s.inputs.push_back(Tensor(inputs[i], "in" + std::to_string(i)));
  s.outputs.push_back(MSTensor("out", mindspore::DataType::kNumberTypeInt8, {}, nullptr, 0, false));
  std::shared_ptr<mindspore::kernel::KernelInterface> iface =
    mindspore::registry::RegisterKernelInterface::GetKernelInterface(provider, &s.prim);
  if (iface == nullptr) iface = std::make_shared<BuiltinInference>();
  const mindspore::Status st = iface->Infer(&s.inputs, &s.outputs, &s.prim);
  if (st == mindspore::kLiteInferInvalid) return -2;
  if (!st.IsOk()) return -1;
  const auto &out = s.outputs[0].Shape();
  for (size_t i = 0; i < out.size() && i < 8; ++i) shape[i] = out[i];
  return static_cast<int32_t>(out.size());
}

void ph_destroy(void *h) { delete static_cast<Session *>(h); }

// 1 when this harness was built with the reference's own RegisterKernel / RegistryKernelImpl, 0 with the stand-in.
int32_t ph_registry_is_real(void) {
#ifdef PH_REAL_REGISTRY_HEADER
  return 1;
#else
  return 0;
#endif
}

// Registry lookup alone, as the scheduler makes it (scheduler.cc:1131-1177): 1 when a creator is registered under
// exactly (arch, provider, data type, op type).
int32_t ph_lookup(const char *arch, const char *provider, int32_t dtype, int32_t op_type) {
  schema::Primitive prim;
  prim.type_ = static_cast<schema::PrimitiveType>(op_type);
  mindspore::registry::KernelDesc desc{static_cast<mindspore::DataType>(dtype), op_type, arch, provider};
  return mindspore::registry::RegisterKernel::GetCreator(&prim, &desc) != nullptr ? 1 : 0;
}

// Registers a creator that declines everything under (arch, provider, dtype, op type); returns the registry's status
// code (0 = registered).
int32_t ph_register_declining(const char *arch, const char *provider, int32_t dtype, int32_t op_type) {
  const auto creator = [](const std::vector<MSTensor> &, const std::vector<MSTensor> &, const schema::Primitive *,
                          const mindspore::Context *) -> std::shared_ptr<mindspore::kernel::Kernel> { return nullptr; };
  const mindspore::Status st = mindspore::registry::RegisterKernel::RegKernel(
    arch, provider, static_cast<mindspore::DataType>(dtype), op_type, creator);
  return st.IsOk() ? 0 : static_cast<int32_t>(st.StatusCode());
}

// 1 when a KernelInterface is registered under `provider` for the operator type, else 0.
int32_t ph_has_provider_interface(const char *provider, int32_t op_type) {
  schema::Primitive prim;
  prim.type_ = static_cast<schema::PrimitiveType>(op_type);
  return mindspore::registry::RegisterKernelInterface::GetKernelInterface(provider, &prim) != nullptr ? 1 : 0;
}

// Registers the harness's own inference class under `provider` for one operator type (see TestInterfaceCreator).
void ph_register_test_interface(const char *provider, int32_t op_type) {
  mindspore::registry::RegisterKernelInterface::Reg(provider, op_type, TestInterfaceCreator);
}

// Two sessions at once: each node is executed `repeats` times on a thread of its own with its own input (the same
// shape it was last run with).  Returns 0, or the first failing stage (of node a in the low byte, node b above it).
int32_t ph_execute_concurrently(void *a, const void *in_a, void *b, const void *in_b, int32_t repeats) {
  int32_t result[2] = {0, 0};
  auto run = [&](void *h, const void *in, int32_t *out) {
    auto *s = static_cast<Session *>(h);
    for (int i = 0; i < repeats && *out == 0; ++i) {
      memcpy(s->inputs[0].MutableData(), in, s->inputs[0].DataSize());
      if (s->kernel->Execute() != 0) *out = kExecuteFailed;
    }
  };
  std::thread ta(run, a, in_a, &result[0]), tb(run, b, in_b, &result[1]);
  ta.join();
  tb.join();
  return result[0] | (result[1] << 8);
}

// The allocator where no page-locked memory can be had (no GPU): Malloc still returns usable, 64-byte-aligned memory
// and the bookkeeping behaves the same.  Returns 0, or the number of the first check that failed.
int32_t ph_allocator_fallback_selftest(void) {
  std::shared_ptr<mindspore::Allocator> a = mindspore::mi355x::MakePinnedAllocator();
  void *p = a->Malloc(1000);
  if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 63) != 0) return 1;
  memset(p, 0x11, 1000);
  if (a->RefCount(p) != 0 || a->SetRefCount(p, 3) != 3 || a->DecRefCount(p, 1) != 2) return 2;
  a->Free(p);
  if (a->RefCount(p) != -1) return 3;
  void *q = a->Malloc(800);
  if (q != p) return 4;  // the freed block is reused
  void *big = a->Malloc(size_t{1} << 20);
  if (big == nullptr) return 5;
  memset(big, 0x22, size_t{1} << 20);
  return 0;  // the destructor releases both
}

// The pinned allocator as the runtime would use it for tensor data (lite::Tensor::MallocData / FreeData with the
// reference counting of the executor).  Returns 0, or the number of the first check that failed.
int32_t ph_allocator_selftest(void) {
  std::shared_ptr<mindspore::Allocator> a = mindspore::mi355x::MakePinnedAllocator();
  void *p = a->Malloc(1000);
  if (p == nullptr) return 1;
  if (a->RefCount(p) != 0 || a->SetRefCount(p, 2) != 2 || a->DecRefCount(p, 1) != 1 || a->IncRefCount(p, 3) != 4) return 2;
  int dummy = 0;
  if (a->RefCount(&dummy) != -1 || a->RefCount(nullptr) != -1 || a->IncRefCount(&dummy, 1) != -1) return 3;
  memset(p, 0x5a, 1000);
  a->Free(p);
  if (a->RefCount(p) != -1) return 4;
  void *q = a->Malloc(900);  // fits the freed block and is not 64 times smaller: reused, count reset
  if (q != p || a->RefCount(q) != 0) return 5;
  void *tiny = a->Malloc(8);  // 1000 > 8 << 6: too wasteful, a new block
  a->Free(q);
  void *tiny2 = a->Malloc(8);
  if (tiny == nullptr || tiny2 == nullptr || tiny2 == q || tiny2 == tiny) return 6;
  void *big = a->Malloc(size_t{1} << 22);
  if (big == nullptr) return 7;
  // the memory is usable by the copies the provider makes
  void *dev = nullptr;
  if (mi_device_malloc(size_t{1} << 22, &dev) != MI_OK) return 8;
  memset(big, 0x3c, size_t{1} << 22);
  void *back = a->Malloc(size_t{1} << 22);
  if (back == nullptr || mi_copy_to_device(dev, big, size_t{1} << 22, nullptr) != MI_OK ||
      mi_copy_to_host(back, dev, size_t{1} << 22, nullptr) != MI_OK || memcmp(big, back, size_t{1} << 22) != 0) {
    return 9;
  }
  mi_device_free(dev);
  a->Free(nullptr);
  a->Free(&dummy);  // unknown pointers are left alone
  return 0;  // everything still allocated is released by the destructor
}
}
