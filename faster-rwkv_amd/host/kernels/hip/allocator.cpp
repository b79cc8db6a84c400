// Caching device allocator behind the Allocator interface (the role of
// kernels/cuda/allocator.cpp:47-474 in the reference).
//
// Design for a 288 GB part and an inference workload: requests fall into two regimes.
//   small (<= 1 MiB): rounded to a power of two and served from per-class free lists;
//     classes are refilled by carving 2 MiB slabs, so thousands of [C]-sized activation
//     vectors cost a handful of hipMalloc calls;
//   large: rounded to 2 MiB and served best-fit from a size-ordered pool of whole
//     device allocations (weights, [T, F] prefill activations).
// Memory is returned to the driver only by Trim().  All device work of the backend is
// issued on one stream, so a block handed out again is ordered after its last use.
#include <cstdio>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "frhip.h"
#include "kernels/allocator.h"
#include "kernels/hip/context.h"
#include "kernels/kernels.h"
#include "kernels/registry.h"

namespace rwkv {
namespace hip {

class CachingAllocator : public Allocator {
public:
  static constexpr size_t kSmallMax = 1u << 20;
  static constexpr size_t kSlab = 2u << 20;
  static constexpr size_t kLargeRound = 2u << 20;

  void *DoAllocate(size_t size) override {
    stream();  // make sure the device is initialised
    std::lock_guard<std::mutex> lock(_mu);
    if (size == 0) size = kAlignSize;
    void *p = size <= kSmallMax ? alloc_small(size) : alloc_large(size);
    RV_CHECK(p != nullptr) << "hip allocator: out of device memory asking for " << size << " bytes";
    return p;
  }

  // Called from tensor destructors: must not throw.  A pointer this allocator did not hand out is
  // reported and dropped.
  void Deallocate(void *ptr) override {
    if (!ptr) return;
    std::lock_guard<std::mutex> lock(_mu);
    auto it = _live.find(ptr);
    if (it == _live.end()) {
      std::fprintf(stderr, "hip allocator: ignoring the release of an unknown pointer %p\n", ptr);
      return;
    }
    const size_t sz = it->second;
    _live.erase(it);
    _in_use -= sz;
    if (sz <= kSmallMax)
      _small[class_of(sz)].push_back(ptr);
    else
      _large.emplace(sz, ptr);
  }

  // Give cached large blocks back to the driver; returns bytes released.
  size_t Trim() {
    std::lock_guard<std::mutex> lock(_mu);
    return release_large_cache();
  }

  size_t reserved() const { return _reserved; }
  size_t in_use() const { return _in_use; }
  size_t driver_calls() const { return _driver_calls; }

private:
  static int class_of(size_t size) {
    int c = 9;  // 512 B
    while ((size_t(1) << c) < size) c++;
    return c;
  }

  size_t release_large_cache() {  // caller holds the mutex
    size_t freed = 0;
    for (auto &kv : _large) {
      frhip_free(kv.second);
      freed += kv.first;
    }
    _large.clear();
    _reserved -= freed;
    return freed;
  }

  void *raw(size_t bytes) {
    void *p = nullptr;
    if (frhip_malloc(&p, bytes) != 0) return nullptr;
    _driver_calls++;
    _reserved += bytes;
    return p;
  }

  void *alloc_small(size_t size) {
    const int c = class_of(size);
    const size_t csz = size_t(1) << c;
    auto &fl = _small[c];
    if (fl.empty()) {
      char *slab = static_cast<char *>(raw(kSlab));
      if (!slab && release_large_cache() > 0) slab = static_cast<char *>(raw(kSlab));  // last resort, as alloc_large
      if (!slab) return nullptr;
      for (size_t off = 0; off + csz <= kSlab; off += csz) fl.push_back(slab + off);
    }
    void *p = fl.back();
    fl.pop_back();
    _live[p] = csz;
    _in_use += csz;
    return p;
  }

  void *alloc_large(size_t size) {
    const size_t rounded = (size + kLargeRound - 1) / kLargeRound * kLargeRound;
    auto it = _large.lower_bound(rounded);
    void *p = nullptr;
    size_t got = rounded;
    // reuse a cached block unless it would waste more than half of itself
    if (it != _large.end() && it->first <= 2 * rounded) {
      p = it->second;
      got = it->first;
      _large.erase(it);
    } else {
      p = raw(rounded);
      if (!p && release_large_cache() > 0) p = raw(rounded);  // last resort: release the cache and retry once
    }
    if (!p) return nullptr;
    _live[p] = got;
    _in_use += got;
    return p;
  }

  std::mutex _mu;
  std::unordered_map<int, std::vector<void *>> _small;
  std::multimap<size_t, void *> _large;
  std::unordered_map<void *, size_t> _live;
  size_t _reserved = 0, _in_use = 0, _driver_calls = 0;
};

static CachingAllocator &instance() {
  static CachingAllocator *a = new CachingAllocator();  // never destroyed: tensors may outlive main()
  return *a;
}

Allocator &allocator() { return instance(); }

void allocator_stats(size_t *reserved, size_t *in_use, size_t *driver_calls) {
  if (reserved) *reserved = instance().reserved();
  if (in_use) *in_use = instance().in_use();
  if (driver_calls) *driver_calls = instance().driver_calls();
}

size_t allocator_trim() { return instance().Trim(); }

KernelRegister allocator_reg("allocator", Device::kHIP, allocator);

}  // namespace hip
}  // namespace rwkv
