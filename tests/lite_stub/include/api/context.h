// TEST INFRASTRUCTURE.  Stand-in for include/api/context.h: the provider only passes the pointer along.
#ifndef TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
#define TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
namespace mindspore {
class Context {};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
