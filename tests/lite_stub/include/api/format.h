// TEST INFRASTRUCTURE.  Stand-in for include/api/format.h (values of mindapi/base/format.h:27-34).
#ifndef TESTS_LITE_STUB_INCLUDE_API_FORMAT_H_
#define TESTS_LITE_STUB_INCLUDE_API_FORMAT_H_
#include <stdint.h>
namespace mindspore {
enum Format : int64_t { NCHW = 0, NHWC = 1, NHWC4 = 2, HWKC = 3, HWCK = 4, KCHW = 5, CKHW = 6, KHWC = 7 };
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_FORMAT_H_
