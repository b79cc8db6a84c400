// Allocator interface of the host layer (reference: kernels/allocator.h:6-15).
// Sizes are rounded up to 512 bytes before they reach DoAllocate.
#pragma once

#include <cstddef>

namespace rwkv {

class Allocator {
public:
  static const int kAlignSize = 512;
  virtual ~Allocator() = default;
  void *Allocate(size_t size) {
    const size_t a = static_cast<size_t>(kAlignSize);
    return DoAllocate((size + a - 1) / a * a);
  }
  virtual void *DoAllocate(size_t size) = 0;
  virtual void Deallocate(void *ptr) = 0;
};

class NullAllocator : public Allocator {
public:
  void *DoAllocate(size_t) override { return nullptr; }
  void Deallocate(void *) override {}
};

inline Allocator &null_allocator() {
  static NullAllocator a;
  return a;
}

}  // namespace rwkv
