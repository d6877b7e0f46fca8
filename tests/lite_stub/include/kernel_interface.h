// TEST INFRASTRUCTURE.  Stand-in for mindspore/lite/include/kernel_interface.h (:29-59).
#ifndef TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
#define TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
#include <memory>
#include <vector>

#include "include/api/status.h"
#include "include/api/types.h"
#include "schema/model_generated.h"

namespace mindspore {
namespace kernel {
class Kernel;
class KernelInterface {
 public:
  virtual ~KernelInterface() = default;
  virtual Status Infer(std::vector<mindspore::MSTensor> *inputs, std::vector<mindspore::MSTensor> *outputs,
                       const schema::Primitive *primitive) {
    return kSuccess;
  }
  virtual Status Infer(std::vector<mindspore::MSTensor> *inputs, std::vector<mindspore::MSTensor> *outputs,
                       const schema::Primitive *primitive, const Kernel *kernel) {
    return Infer(inputs, outputs, primitive);
  }
};
}  // namespace kernel
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
