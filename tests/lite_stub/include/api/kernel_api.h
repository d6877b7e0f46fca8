// TEST INFRASTRUCTURE.  Stand-in for include/api/kernel_api.h, cut down to what a provider kernel touches: the three
// life-cycle calls the runtime makes and the protected tensor lists (reference: MSKernel :29-140, IKernel :143-166).
#ifndef TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#define TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
#include <vector>

#include "include/api/status.h"
#include "include/api/types.h"

namespace mindspore {
class Context;
namespace kernel {
class MSKernel {
 public:
  virtual ~MSKernel() = default;
  virtual int Prepare() = 0;
  virtual int ReSize() = 0;
  virtual int Execute() = 0;

 protected:
  MSKernel() = default;
  MSKernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const Context *ctx)
      : context_(ctx), inputs_(in), outputs_(out) {}
  const Context *context_ = nullptr;
  std::vector<MSTensor> inputs_, outputs_;
};

template <typename Primitive>
class IKernel : public MSKernel {
 protected:
  IKernel() = default;
  IKernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const Primitive *primitive,
          const Context *ctx)
      : MSKernel(in, out, ctx), primitive_(primitive) {}
  const Primitive *primitive_ = nullptr;
};
}  // namespace kernel
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_KERNEL_API_H_
