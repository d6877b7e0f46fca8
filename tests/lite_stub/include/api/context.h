// TEST INFRASTRUCTURE.  Stand-in for include/api/context.h: the provider passes the pointer along and asks whether the
// session runs its nodes in parallel.
#ifndef TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
#define TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
namespace mindspore {
class Context {
 public:
  void SetEnableParallel(bool is_parallel) { enable_parallel_ = is_parallel; }
  bool GetEnableParallel() const { return enable_parallel_; }

 private:
  bool enable_parallel_ = false;
};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_CONTEXT_H_
