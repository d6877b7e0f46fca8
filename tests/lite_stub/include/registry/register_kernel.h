// TEST INFRASTRUCTURE.  Stand-in for mindspore/lite/include/registry/register_kernel.h (:34-102): the same
// registration call, kept in a process-wide table that the harness queries the way the scheduler does
// (exact match on arch, provider, data type and op type; scheduler.cc:1131-1177).
//
// Where the reference tree is at hand the harness is built with the reference's OWN registry instead: its header
// (named by PH_REAL_REGISTRY_HEADER on the compiler's command line) and its sources register_kernel.cc /
// register_kernel_impl.cc, compiled from where they lie (tests/lite_stub/build.py).  The table below is then unused.
#ifdef PH_REAL_REGISTRY_HEADER
#include PH_REAL_REGISTRY_HEADER
#endif
#ifndef PH_REAL_REGISTRY_HEADER
#ifndef TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_H_
#define TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_H_
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "include/api/context.h"
#include "include/api/data_type.h"
#include "include/api/kernel.h"
#include "include/api/status.h"
#include "include/api/types.h"
#include "schema/model_generated.h"

namespace mindspore {
namespace registry {
struct KernelDesc {
  DataType data_type;
  int type;
  std::string arch;
  std::string provider;
};
using CreateKernel = std::function<std::shared_ptr<kernel::Kernel>(
  const std::vector<MSTensor> &inputs, const std::vector<MSTensor> &outputs, const schema::Primitive *primitive,
  const mindspore::Context *ctx)>;

class RegisterKernel {
 public:
  using Key = std::tuple<std::string, std::string, int, int>;
  static std::map<Key, CreateKernel> &Table() {
    static std::map<Key, CreateKernel> table;
    return table;
  }
  static Status RegKernel(const std::string &arch, const std::string &provider, DataType data_type, int type,
                          const CreateKernel creator) {
    Table()[Key(arch, provider, static_cast<int>(data_type), type)] = creator;
    return kSuccess;
  }
  static CreateKernel GetCreator(const schema::Primitive *primitive, KernelDesc *desc) {
    auto it = Table().find(Key(desc->arch, desc->provider, static_cast<int>(desc->data_type), desc->type));
    return it == Table().end() ? nullptr : it->second;
  }
};
}  // namespace registry
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_REGISTRY_REGISTER_KERNEL_H_
#endif  // PH_REAL_REGISTRY_HEADER
