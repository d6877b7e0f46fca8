// TEST INFRASTRUCTURE.  Stand-in for mindspore/lite/include/registry/register_kernel_interface.h (:33-75).
#ifndef TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_INTERFACE_H_
#define TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_INTERFACE_H_
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <utility>

#include "include/kernel_interface.h"
#include "schema/model_generated.h"

namespace mindspore {
namespace registry {
using KernelInterfaceCreator = std::function<std::shared_ptr<kernel::KernelInterface>()>;
class RegisterKernelInterface {
 public:
  static std::map<std::pair<std::string, int>, KernelInterfaceCreator> &Table() {
    static std::map<std::pair<std::string, int>, KernelInterfaceCreator> table;
    return table;
  }
  static Status Reg(const std::string &provider, int op_type, const KernelInterfaceCreator creator) {
    Table()[std::make_pair(provider, op_type)] = creator;
    return kSuccess;
  }
  static std::shared_ptr<kernel::KernelInterface> GetKernelInterface(const std::string &provider,
                                                                     const schema::Primitive *primitive,
                                                                     const kernel::Kernel *kernel = nullptr) {
    auto it = Table().find(std::make_pair(provider, static_cast<int>(primitive->value_type())));
    return it == Table().end() ? nullptr : it->second();
  }
};
}  // namespace registry
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_INTERFACE_H_
