// TEST INFRASTRUCTURE.  Stand-in for include/api/allocator.h: the abstract interface (:25-99) an allocator installed
// with DeviceInfoContext::SetAllocator implements.
#ifndef TESTS_LITE_STUB_INCLUDE_API_ALLOCATOR_H_
#define TESTS_LITE_STUB_INCLUDE_API_ALLOCATOR_H_
#include <stddef.h>

#include <memory>

namespace mindspore {
class Allocator {
 public:
  virtual ~Allocator() = default;
  virtual void *Malloc(size_t size) = 0;
  virtual void Free(void *ptr) = 0;
  virtual int RefCount(void *ptr) = 0;
  virtual int SetRefCount(void *ptr, int ref_count) = 0;
  virtual int DecRefCount(void *ptr, int ref_count) = 0;
  virtual int IncRefCount(void *ptr, int ref_count) = 0;
  virtual void *Prepare(void *ptr) { return ptr; }
};
}  // namespace mindspore
#endif  // TESTS_LITE_STUB_INCLUDE_API_ALLOCATOR_H_
