// Caching device allocator behind the Allocator interface (the role of
// kernels/cuda/allocator.cpp:47-474 in the reference).
//
// Design for a 288 GB part and an inference workload: requests fall into two regimes.
//   small (<= 1 MiB): rounded to a power of two and served from per-class free lists;
//     classes are refilled by carving 2 MiB slabs, so thousands of [C]-sized activation
//     vectors cost a handful of hipMalloc calls;
//   large: rounded to 2 MiB and served best-fit from the free blocks of the driver
//     allocations made so far ("segments": weights, [T, F] prefill activations).  A free
//     block that is at least twice the request, or would leave 128 MiB or more unused, is
//     split and its tail stays free (kernels/cuda/allocator.cpp:267-268); a released block
//     merges with free neighbours of its segment (kernels/cuda/allocator.cpp:449-459), so
//     prompts of changing length keep being served from the memory of the longest one.
// Memory is returned to the driver only by Trim() (segments that are free as a whole).
// All device work of the backend is issued on one stream, so a block handed out again is
// ordered after its last use.
#include <cstdio>
#include <map>
#include <set>
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
  static constexpr size_t kSplitRemainder = 128u << 20;  // kernels/cuda/allocator.cpp:28 (kPieceSplitThreshold)

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
      free_large(static_cast<char *>(ptr));
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

  // A block of a large segment.  Blocks of one segment tile it without gaps, in address order.
  struct Block {
    size_t size;
    char *segment;  // start of the driver allocation this block is part of
    bool free;
  };
  using BlockMap = std::map<char *, Block>;

  // Release every segment that is one free block again; caller holds the mutex.
  size_t release_large_cache() {
    size_t freed = 0;
    for (auto it = _blocks.begin(); it != _blocks.end();) {
      const auto seg = _segments.find(it->first);
      if (it->second.free && seg != _segments.end() && seg->second == it->second.size) {
        _free_by_size.erase({it->second.size, it->first});
        frhip_free(it->first);
        freed += it->second.size;
        _segments.erase(seg);
        it = _blocks.erase(it);
      } else {
        ++it;
      }
    }
    _reserved -= freed;
    return freed;
  }

  // Mark a large block free and merge it with free neighbours of the same segment.
  void free_large(char *ptr) {
    auto it = _blocks.find(ptr);
    if (it == _blocks.end()) return;
    it->second.free = true;
    auto next = std::next(it);
    if (next != _blocks.end() && next->second.free && next->second.segment == it->second.segment) {
      _free_by_size.erase({next->second.size, next->first});
      it->second.size += next->second.size;
      _blocks.erase(next);
    }
    if (it != _blocks.begin()) {
      auto prev = std::prev(it);
      if (prev->second.free && prev->second.segment == it->second.segment) {
        _free_by_size.erase({prev->second.size, prev->first});
        prev->second.size += it->second.size;
        _blocks.erase(it);
        it = prev;
      }
    }
    _free_by_size.insert({it->second.size, it->first});
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
    BlockMap::iterator blk = _blocks.end();
    auto fit = _free_by_size.lower_bound({rounded, nullptr});  // best fit: the smallest free block that is large enough
    if (fit != _free_by_size.end()) {
      blk = _blocks.find(fit->second);
      _free_by_size.erase(fit);
    } else {
      char *p = static_cast<char *>(raw(rounded));
      if (!p && release_large_cache() > 0) p = static_cast<char *>(raw(rounded));  // last resort: release the cache and retry once
      if (!p) return nullptr;
      _segments[p] = rounded;
      blk = _blocks.emplace(p, Block{rounded, p, true}).first;
    }
    Block &b = blk->second;
    if (b.size >= 2 * rounded || b.size - rounded >= kSplitRemainder) {  // the tail stays in the pool
      char *tail = blk->first + rounded;
      _blocks.emplace(tail, Block{b.size - rounded, b.segment, true});
      _free_by_size.insert({b.size - rounded, tail});
      b.size = rounded;
    }
    b.free = false;
    _live[blk->first] = b.size;
    _in_use += b.size;
    return blk->first;
  }

  std::mutex _mu;
  std::unordered_map<int, std::vector<void *>> _small;
  BlockMap _blocks;                                  // every block of every large segment, by address
  std::set<std::pair<size_t, char *>> _free_by_size;  // the free ones, by size then address
  std::map<char *, size_t> _segments;                // driver allocations of the large regime: start -> bytes
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
