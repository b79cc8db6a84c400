// CPU-side operators the host path needs around a device model: the allocator,
// fill_ and cast_dtype used by Model::ResetStates and by tests (reference:
// kernels/cpu/allocator.cpp:8-28, fill.cpp:9-27, cast_dtype.cpp:9-29).  The model's
// arithmetic is not implemented for the CPU here.
#include <cstdlib>
#include <new>

#include "kernels/kernels.h"
#include "kernels/registry.h"

namespace rwkv {
namespace cpu {

class HostAllocator : public Allocator {
public:
  void *DoAllocate(size_t size) override {
    if (size == 0) size = kAlignSize;
    void *p = std::aligned_alloc(kAlignSize, size);
    if (!p) throw std::bad_alloc();
    return p;
  }
  void Deallocate(void *ptr) override { std::free(ptr); }
};

Allocator &allocator() {
  static HostAllocator a;
  return a;
}

Tensor &fill_(Tensor &x, float value) {
  const LengthType n = x.numel();
  if (x.dtype() == DType::kFloat32) {
    float *p = x.data_ptr<float>();
    for (LengthType i = 0; i < n; i++) p[i] = value;
  } else if (x.dtype() == DType::kFloat16) {
    float16 *p = x.data_ptr<float16>();
    const float16 v(value);
    for (LengthType i = 0; i < n; i++) p[i] = v;
  } else {
    RV_UNIMPLEMENTED();
  }
  return x;
}

Tensor cast_dtype(const Tensor &x, DType dtype) {
  if (x.dtype() == dtype) return x;
  Tensor y = Tensor::Empty(x.shape(), dtype, Device::kCPU);
  const LengthType n = x.numel();
  if (x.dtype() == DType::kFloat16 && dtype == DType::kFloat32) {
    const float16 *s = x.data_ptr<float16>();
    float *d = y.data_ptr<float>();
    for (LengthType i = 0; i < n; i++) d[i] = static_cast<float>(s[i]);
  } else if (x.dtype() == DType::kFloat32 && dtype == DType::kFloat16) {
    const float *s = x.data_ptr<float>();
    float16 *d = y.data_ptr<float16>();
    for (LengthType i = 0; i < n; i++) d[i] = float16(s[i]);
  } else {
    RV_UNIMPLEMENTED();
  }
  return y;
}

KernelRegister allocator_reg("allocator", Device::kCPU, allocator);
KernelRegister fill_reg("fill_", Device::kCPU, fill_);
KernelRegister cast_reg("cast_dtype", Device::kCPU, cast_dtype);

}  // namespace cpu
}  // namespace rwkv
