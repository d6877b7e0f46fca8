// TEST INFRASTRUCTURE.  Minimal stand-in for MindSpore's include/api/status.h: the status codes the provider returns
// (numeric values as in the reference, include/api/status.h:32-123) and a Status that converts from them.
#ifndef TESTS_LITE_STUB_INCLUDE_API_STATUS_H_
#define TESTS_LITE_STUB_INCLUDE_API_STATUS_H_
#include <stdint.h>

#include <functional>
#include <string>
#include <vector>

#ifndef MS_API
#define MS_API
#endif

namespace mindspore {
// the string <-> char-vector helpers of include/api/dual_abi_helper.h that the registration headers use
inline std::vector<char> StringToChar(const std::string &s) { return std::vector<char>(s.begin(), s.end()); }
inline std::string CharToString(const std::vector<char> &c) { return std::string(c.begin(), c.end()); }

enum CompCode : uint32_t { kCore = 0x00000000u, kLite = 0xF0000000u };
enum StatusCode : uint32_t {
  kSuccess = 0,
  kLiteError = kLite | (0x0FFFFFFF & -1),
  kLiteNullptr = kLite | (0x0FFFFFFF & -2),
  kLiteParamInvalid = kLite | (0x0FFFFFFF & -3),
  kLiteMemoryFailed = kLite | (0x0FFFFFFF & -6),
  kLiteNotSupport = kLite | (0x0FFFFFFF & -7),
  kLiteInferError = kLite | (0x0FFFFFFF & -500),
  kLiteInferInvalid = kLite | (0x0FFFFFFF & -501),
};
class Status {
 public:
  Status() = default;
  Status(enum StatusCode code) : code_(code) {}  // NOLINT(runtime/explicit)
  enum StatusCode StatusCode() const { return code_; }
  bool operator==(enum StatusCode other) const { return code_ == other; }
  bool operator!=(enum StatusCode other) const { return code_ != other; }
  bool IsOk() const { return code_ == kSuccess; }

 private:
  enum StatusCode code_ = kSuccess;
};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_STATUS_H_
