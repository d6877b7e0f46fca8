// TEST INFRASTRUCTURE.  Stand-in for include/api/kernel.h (:29-55): kernel::Kernel over schema::Primitive.
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
  Kernel() = default;
  Kernel(const std::vector<mindspore::MSTensor> &inputs, const std::vector<mindspore::MSTensor> &outputs,
         const schema::Primitive *primitive, const mindspore::Context *ctx)
      : IKernel<schema::Primitive>(inputs, outputs, primitive, ctx) {
    if (primitive != nullptr) type_ = primitive->value_type();
  }
  virtual ~Kernel() = default;
  virtual schema::PrimitiveType type() const { return type_; }
  virtual schema::QuantType quant_type() const { return quant_type_; }

 protected:
  schema::PrimitiveType type_ = schema::PrimitiveType_NONE;
  schema::QuantType quant_type_ = schema::QuantType_QUANT_NONE;  // never populated by the runtime either
};
}  // namespace mindspore::kernel
#endif  // TESTS_LITE_STUB_INCLUDE_API_KERNEL_H_
