// TEST INFRASTRUCTURE.  Stand-in for the header that flatc generates from MindSpore Lite's schema
// (mindspore/lite/schema/{model,ops,ops_types}.fbs), written by hand for the handful of tables the provider reads:
// the same names, accessor signatures and enum values, backed by plain structs instead of a flatbuffer.  It lets
// mindspore_amd/provider/mi355x_provider.cc be compiled (and, with the other stand-ins in this directory, run) in an
// image that has neither flatc nor a Lite SDK.  Not a substitute for building against the real SDK.
#ifndef TESTS_LITE_STUB_SCHEMA_MODEL_GENERATED_H_
#define TESTS_LITE_STUB_SCHEMA_MODEL_GENERATED_H_

#include <stdint.h>

#include <string>
#include <vector>

namespace flatbuffers {
template <typename T>
class Vector {
 public:
  Vector() = default;
  explicit Vector(std::vector<T> v) : v_(std::move(v)) {}
  uint32_t size() const { return static_cast<uint32_t>(v_.size()); }
  T Get(uint32_t i) const { return v_[i]; }

 private:
  std::vector<T> v_;
};
}  // namespace flatbuffers

namespace mindspore {
namespace schema {
// positions in `union PrimitiveType` of ops.fbs
enum PrimitiveType : int {
  PrimitiveType_NONE = 0,
  PrimitiveType_Conv2DFusion = 35,
  PrimitiveType_FullConnection = 67,
  PrimitiveType_MatMulFusion = 89,
  PrimitiveType_Custom = 191,
  PrimitiveType_DynamicQuant = 203,
  PrimitiveType_FillV2 = 221,  // the union's last member
  PrimitiveType_MIN = PrimitiveType_NONE,
  PrimitiveType_MAX = PrimitiveType_FillV2,
};
enum QuantType : int {  // model.fbs:76-84
  QuantType_QUANT_NONE = 0,
  QuantType_QUANT_WEIGHT = 4,
  QuantType_QUANT_ALL = 5,
  QuantType_QUANT_DYNAMIC = 6,
};
enum ActivationType : int8_t {  // ops_types.fbs:62-66
  ActivationType_NO_ACTIVATION = 0,
  ActivationType_RELU = 1,
  ActivationType_RELU6 = 3,
};
enum PadMode : int8_t { PadMode_PAD = 0, PadMode_SAME = 1, PadMode_VALID = 2 };  // ops_types.fbs:111-115

struct MatMulFusion {  // ops.fbs:713-717
  bool transpose_a_ = false, transpose_b_ = false;
  ActivationType activation_type_ = ActivationType_NO_ACTIVATION;
  bool transpose_a() const { return transpose_a_; }
  bool transpose_b() const { return transpose_b_; }
  ActivationType activation_type() const { return activation_type_; }
};

struct FullConnection {  // ops.fbs:601-606
  bool has_bias_ = false, use_axis_ = false;
  int64_t axis_ = 0;
  ActivationType activation_type_ = ActivationType_NO_ACTIVATION;
  bool has_bias() const { return has_bias_; }
  bool use_axis() const { return use_axis_; }
  int64_t axis() const { return axis_; }
  ActivationType activation_type() const { return activation_type_; }
};

struct Conv2DFusion {  // ops.fbs:437-449
  flatbuffers::Vector<int64_t> kernel_size_, stride_, dilation_, pad_list_;
  bool has_kernel_size_ = true, has_stride_ = true, has_dilation_ = true, has_pad_list_ = true;
  PadMode pad_mode_ = PadMode_PAD;
  int64_t group_ = 1, in_channel_ = 0, out_channel_ = 0;
  ActivationType activation_type_ = ActivationType_NO_ACTIVATION;
  const flatbuffers::Vector<int64_t> *kernel_size() const { return has_kernel_size_ ? &kernel_size_ : nullptr; }
  const flatbuffers::Vector<int64_t> *stride() const { return has_stride_ ? &stride_ : nullptr; }
  const flatbuffers::Vector<int64_t> *dilation() const { return has_dilation_ ? &dilation_ : nullptr; }
  const flatbuffers::Vector<int64_t> *pad_list() const { return has_pad_list_ ? &pad_list_ : nullptr; }
  PadMode pad_mode() const { return pad_mode_; }
  int64_t group() const { return group_; }
  int64_t in_channel() const { return in_channel_; }
  int64_t out_channel() const { return out_channel_; }
  ActivationType activation_type() const { return activation_type_; }
};

struct DynamicQuant {  // ops.fbs:1248-1255
  bool symmetric_ = false;
  int64_t dst_type_ = 32;
  flatbuffers::Vector<int32_t> prefer_axes_;
  bool has_prefer_axes_ = false;
  bool symmetric() const { return symmetric_; }
  int64_t dst_type() const { return dst_type_; }
  const flatbuffers::Vector<int32_t> *prefer_axes() const { return has_prefer_axes_ ? &prefer_axes_ : nullptr; }
};

struct String {  // flatbuffers::String, as far as the kernel registry reads it
  std::string s_;
  std::string str() const { return s_; }
};

struct Custom {  // ops.fbs: table Custom { type: string; attr: [Attribute]; }
  String type_;
  const String *type() const { return &type_; }
};

struct Primitive {  // model.fbs:86-88 (a union in the real schema: exactly one member is meaningful)
  PrimitiveType type_ = PrimitiveType_NONE;
  MatMulFusion matmul_;
  FullConnection fc_;
  Conv2DFusion conv_;
  DynamicQuant dynquant_;
  Custom custom_;
  PrimitiveType value_type() const { return type_; }
  const Custom *value_as_Custom() const { return type_ == PrimitiveType_Custom ? &custom_ : nullptr; }
  const MatMulFusion *value_as_MatMulFusion() const { return type_ == PrimitiveType_MatMulFusion ? &matmul_ : nullptr; }
  const FullConnection *value_as_FullConnection() const {
    return type_ == PrimitiveType_FullConnection ? &fc_ : nullptr;
  }
  const Conv2DFusion *value_as_Conv2DFusion() const { return type_ == PrimitiveType_Conv2DFusion ? &conv_ : nullptr; }
  const DynamicQuant *value_as_DynamicQuant() const { return type_ == PrimitiveType_DynamicQuant ? &dynquant_ : nullptr; }
};
}  // namespace schema
}  // namespace mindspore

#endif  // TESTS_LITE_STUB_SCHEMA_MODEL_GENERATED_H_
