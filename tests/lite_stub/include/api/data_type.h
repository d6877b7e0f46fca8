// TEST INFRASTRUCTURE.  Stand-in for include/api/data_type.h (numeric ids as in the reference, :22-42).
#ifndef TESTS_LITE_STUB_INCLUDE_API_DATA_TYPE_H_
#define TESTS_LITE_STUB_INCLUDE_API_DATA_TYPE_H_
namespace mindspore {
enum class DataType : int {
  kTypeUnknown = 0,
  kNumberTypeBegin = 29,
  kNumberTypeInt8 = 32,
  kNumberTypeInt32 = 34,
  kNumberTypeUInt8 = 37,
  kNumberTypeFloat32 = 43,
  kNumberTypeEnd = 52,
};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_DATA_TYPE_H_
