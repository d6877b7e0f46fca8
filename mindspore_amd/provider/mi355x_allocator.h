// A mindspore::Allocator (include/api/allocator.h:25-99) that hands out page-locked host memory from
// libmi355x_int8.so, for DeviceInfoContext::SetAllocator (include/api/context.h:217) of the CPU device info the
// mi355x provider runs under: tensors allocated through it (graph inputs and outputs, activations between builtin
// kernels) are then copied to and from the GPU by DMA without the runtime's bounce buffer.
//
//   auto cpu = std::make_shared<mindspore::CPUDeviceInfo>();
//   cpu->SetProvider("mi355x");
//   cpu->SetProviderDevice("CPU");
//   cpu->SetAllocator(mindspore::mi355x::MakePinnedAllocator());
//
// Same contract as Lite's DefaultAllocator (mindspore/lite/src/litert/inner_allocator.cc:51-175): a freed block goes
// to a size-ordered free list and is reused for requests it fits without being more than 2^6 times too large
// (shiftFactor_, inner_allocator.h), reference counts start at 0 and are -1 for pointers the allocator does not
// know.  Blocks return to the system when the allocator is destroyed.  Thread safe.
#ifndef MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
#define MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
#include <stddef.h>
#include <stdint.h>

#include <map>
#include <memory>
#include <mutex>
#include <unordered_map>

#include "include/api/allocator.h"
#include "mi355x_int8.h"

namespace mindspore {
namespace mi355x {
class PinnedAllocator : public Allocator {
 public:
  PinnedAllocator() = default;
  PinnedAllocator(const PinnedAllocator &) = delete;
  PinnedAllocator &operator=(const PinnedAllocator &) = delete;
  ~PinnedAllocator() override {
    for (auto &it : allocated_) mi_host_free(it.first);
    for (auto &it : free_) mi_host_free(it.second);
  }

  void *Malloc(size_t size) override {
    if (size == 0) size = 1;
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = free_.lower_bound(size);
    if (it != free_.end() && it->first <= (size >= (SIZE_MAX >> kReuseShift) ? SIZE_MAX : size << kReuseShift)) {
      void *p = it->second;
      allocated_[p] = Block{it->first, 0};
      free_.erase(it);
      return p;
    }
    void *p = nullptr;
    if (mi_host_malloc(size, &p) != MI_OK) return nullptr;
    allocated_[p] = Block{size, 0};
    return p;
  }

  void Free(void *ptr) override {
    if (ptr == nullptr) return;
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = allocated_.find(ptr);
    if (it == allocated_.end()) return;  // not ours: nothing this allocator may release
    free_.emplace(it->second.size, ptr);
    allocated_.erase(it);
  }

  int RefCount(void *ptr) override { return Update(ptr, [](int r) { return r; }); }
  int SetRefCount(void *ptr, int ref_count) override { return Update(ptr, [=](int) { return ref_count; }); }
  int DecRefCount(void *ptr, int ref_count) override { return Update(ptr, [=](int r) { return r - ref_count; }); }
  int IncRefCount(void *ptr, int ref_count) override { return Update(ptr, [=](int r) { return r + ref_count; }); }

 private:
  struct Block {
    size_t size;
    int ref_count;
  };
  static constexpr int kReuseShift = 6;

  template <typename F>
  int Update(void *ptr, F f) {
    if (ptr == nullptr) return -1;
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = allocated_.find(ptr);
    if (it == allocated_.end()) return -1;
    it->second.ref_count = f(it->second.ref_count);
    return it->second.ref_count;
  }

  std::mutex mutex_;
  std::unordered_map<void *, Block> allocated_;
  std::multimap<size_t, void *> free_;
};

inline std::shared_ptr<Allocator> MakePinnedAllocator() { return std::make_shared<PinnedAllocator>(); }
}  // namespace mi355x
}  // namespace mindspore
#endif  // MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
