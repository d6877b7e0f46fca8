// TEST INFRASTRUCTURE.  Stand-in for mindspore/lite/include/kernel_interface.h: the one virtual a provider overrides
// to answer shape inference (reference :29-59, which also has an overload that receives the kernel).
#ifndef TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
#define TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
#include <vector>

#include "include/api/status.h"
#include "include/api/types.h"
#include "schema/model_generated.h"

namespace mindspore::kernel {
class KernelInterface {
 public:
  virtual ~KernelInterface() = default;
  virtual Status Infer(std::vector<MSTensor> *inputs, std::vector<MSTensor> *outputs, const schema::Primitive *prim) = 0;
};
}  // namespace mindspore::kernel
#endif  // TESTS_LITE_STUB_INCLUDE_KERNEL_INTERFACE_H_
