// TEST INFRASTRUCTURE.  Stand-in for include/api/kernel.h: the base class a provider kernel derives from, bound to
// the schema's Primitive.  Only construction is needed here; the reference class (:29-55) also carries the op and
// quant type, which no provider kernel of this repository reads.
#ifndef TESTS_LITE_STUB_INCLUDE_API_KERNEL_H_
#define TESTS_LITE_STUB_INCLUDE_API_KERNEL_H_
#include <vector>

#include "include/api/context.h"
#include "include/api/kernel_api.h"
#include "include/api/types.h"
#include "schema/model_generated.h"

namespace mindspore::kernel {
class Kernel : public IKernel<schema::Primitive> {
 public:
  Kernel(const std::vector<MSTensor> &in, const std::vector<MSTensor> &out, const schema::Primitive *prim,
         const Context *ctx)
      : IKernel<schema::Primitive>(in, out, prim, ctx) {}
};
}  // namespace mindspore::kernel
#endif  // TESTS_LITE_STUB_INCLUDE_API_KERNEL_H_
