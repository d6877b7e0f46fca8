// TEST INFRASTRUCTURE.  Stand-in for the part of include/api/types.h the provider uses: QuantParam (:55-61) and an
// MSTensor with the same accessors (:165-315), backed by host memory.  Like the real class it is a handle: copies share
// one tensor, so what a kernel writes through its copy (data, quant params, shape) is seen by the harness.
#ifndef TESTS_LITE_STUB_INCLUDE_API_TYPES_H_
#define TESTS_LITE_STUB_INCLUDE_API_TYPES_H_
#include <stdint.h>

#include <memory>
#include <string>
#include <vector>

#include "include/api/data_type.h"
#include "include/api/format.h"
#include "include/api/status.h"

namespace mindspore {
struct QuantParam {
  int bit_num;
  double scale;
  int32_t zero_point;
  double min;
  double max;
};

class MSTensor {
 public:
  struct Impl {
    std::string name;
    enum DataType dtype = DataType::kTypeUnknown;
    std::vector<int64_t> shape;
    mindspore::Format format = NHWC;
    std::shared_ptr<std::vector<char>> data;  // null until allocated
    std::vector<QuantParam> quant;
    bool is_const = false;
    void *device_data = nullptr;  // an address only: the tensor never frees it (lite::Tensor::device_data_)
  };
  MSTensor() : impl_(std::make_shared<Impl>()) {}
  // harness-side constructor (the real class is created by the runtime)
  MSTensor(const std::string &name, enum DataType dtype, const std::vector<int64_t> &shape, const void *data,
           size_t bytes, bool is_const)
      : impl_(std::make_shared<Impl>()) {
    impl_->name = name;
    impl_->dtype = dtype;
    impl_->shape = shape;
    impl_->is_const = is_const;
    if (data != nullptr) {
      const char *p = static_cast<const char *>(data);
      impl_->data = std::make_shared<std::vector<char>>(p, p + bytes);
    }
  }

  enum DataType DataType() const { return impl_->dtype; }
  const std::vector<int64_t> &Shape() const { return impl_->shape; }
  int64_t ElementNum() const {
    int64_t n = 1;
    for (int64_t d : impl_->shape) n *= d;
    return n;
  }
  size_t DataSize() const { return static_cast<size_t>(ElementNum()) * ElementSize(); }
  std::shared_ptr<const void> Data() const {
    if (impl_->data == nullptr) return nullptr;
    return std::shared_ptr<const void>(impl_->data, impl_->data->data());
  }
  void *MutableData() {  // allocates on first use, as lite::Tensor::MallocData does
    if (impl_->data == nullptr || impl_->data->size() != DataSize()) {
      impl_->data = std::make_shared<std::vector<char>>(DataSize());
    }
    return impl_->data->data();
  }
  bool IsConst() const { return impl_->is_const; }
  void SetShape(const std::vector<int64_t> &shape) { impl_->shape = shape; }
  void SetFormat(mindspore::Format format) { impl_->format = format; }
  mindspore::Format format() const { return impl_->format; }
  std::vector<QuantParam> QuantParams() const { return impl_->quant; }
  void SetQuantParams(std::vector<QuantParam> quant_params) { impl_->quant = std::move(quant_params); }
  std::string Name() const { return impl_->name; }
  bool operator==(const MSTensor &tensor) const { return impl_ == tensor.impl_; }
  void SetDeviceData(void *data) { impl_->device_data = data; }
  void *GetDeviceData() { return impl_->device_data; }
  bool HasHostData() const { return impl_->data != nullptr; }  // harness-side

 private:
  size_t ElementSize() const {
    switch (impl_->dtype) {
      case DataType::kNumberTypeInt32:
      case DataType::kNumberTypeFloat32:
        return 4;
      default:
        return 1;
    }
  }
  std::shared_ptr<Impl> impl_;
};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_TYPES_H_
