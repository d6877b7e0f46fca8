// TEST INFRASTRUCTURE.  Stand-in for include/api/kernel_api.h: MSKernel (:29-140) and IKernel (:143-166) with the
// members a provider kernel touches.
#ifndef TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#define TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#include <string>
#include <utility>
#include <vector>

#include "include/api/status.h"
#include "include/api/types.h"

namespace mindspore {
class Context;
namespace kernel {
class MSKernel {
 public:
  MSKernel() = default;
  MSKernel(std::vector<mindspore::MSTensor> inputs, std::vector<mindspore::MSTensor> outputs,
           const mindspore::Context *ctx)
      : context_(ctx), inputs_(std::move(inputs)), outputs_(std::move(outputs)) {}
  virtual ~MSKernel() = default;
  virtual int InferShape() { return kLiteError; }
  virtual int Prepare() = 0;
  virtual int Execute() = 0;
  virtual int ReSize() = 0;
  virtual void set_inputs(const std::vector<mindspore::MSTensor> &in_tensors) { inputs_ = in_tensors; }
  virtual void set_outputs(const std::vector<mindspore::MSTensor> &out_tensors) { outputs_ = out_tensors; }
  virtual const std::vector<mindspore::MSTensor> &inputs() { return inputs_; }
  virtual const std::vector<mindspore::MSTensor> &outputs() { return outputs_; }
  const mindspore::Context *context() const { return context_; }

 protected:
  std::string name_;
  const mindspore::Context *context_ = nullptr;
  std::vector<mindspore::MSTensor> inputs_;
  std::vector<mindspore::MSTensor> outputs_;
};

template <typename Primitive>
class IKernel : public MSKernel {
 public:
  IKernel() = default;
  IKernel(const std::vector<mindspore::MSTensor> &inputs, const std::vector<mindspore::MSTensor> &outputs,
          const Primitive *primitive, const mindspore::Context *ctx)
      : MSKernel(inputs, outputs, ctx), primitive_(primitive) {}
  ~IKernel() override = default;
  const Primitive *primitive() const { return primitive_; }

 protected:
  const Primitive *primitive_ = nullptr;
};
}  // namespace kernel
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
