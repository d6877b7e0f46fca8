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
// The allocator initialises the library itself (a session may allocate tensors before any creator of the provider
// has run, or run a model that has none of its operators); where page-locked memory cannot be had -- no GPU, no
// gfx950 -- it hands out ordinary 64-byte-aligned memory, so that a CPU-only session keeps working.
#ifndef MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
#define MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

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
    for (auto &it : allocated_) Release(it.first, it.second.pinned);
    for (auto &it : free_) Release(it.second.ptr, it.second.pinned);
  }

  void *Malloc(size_t size) override {
    if (size == 0) size = 1;
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = free_.lower_bound(size);
    if (it != free_.end() && it->first <= (size >= (SIZE_MAX >> kReuseShift) ? SIZE_MAX : size << kReuseShift)) {
      void *p = it->second.ptr;
      allocated_[p] = Block{it->first, 0, it->second.pinned};
      free_.erase(it);
      return p;
    }
    void *p = nullptr;
    bool pinned = false;
    if (LibraryUp() && mi_host_malloc(size, &p) == MI_OK) {
      pinned = true;
    } else if (posix_memalign(&p, 64, (size + 63) & ~size_t{63}) != 0) {
      return nullptr;
    }
    allocated_[p] = Block{size, 0, pinned};
    return p;
  }

  void Free(void *ptr) override {
    if (ptr == nullptr) return;
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = allocated_.find(ptr);
    if (it == allocated_.end()) return;  // not ours: nothing this allocator may release
    free_.emplace(it->second.size, FreeBlock{ptr, it->second.pinned});
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
    bool pinned;  // from mi_host_malloc (else from posix_memalign)
  };
  struct FreeBlock {
    void *ptr;
    bool pinned;
  };
  static constexpr int kReuseShift = 6;

  // the same device choice as the provider's kernels make (MI355X_DEVICE, else device 0)
  static bool LibraryUp() {
    static const bool ok = [] {
      const char *device = getenv("MI355X_DEVICE");
      return mi_init(device != nullptr ? atoi(device) : 0) == MI_OK;
    }();
    return ok;
  }
  static void Release(void *p, bool pinned) {
    if (pinned) {
      mi_host_free(p);
    } else {
      free(p);
    }
  }

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
  std::multimap<size_t, FreeBlock> free_;
};

inline std::shared_ptr<Allocator> MakePinnedAllocator() { return std::make_shared<PinnedAllocator>(); }
}  // namespace mi355x
}  // namespace mindspore
#endif  // MINDSPORE_AMD_PROVIDER_MI355X_ALLOCATOR_H_
