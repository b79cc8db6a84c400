// Tensor, storage, dtype and device enums of the host layer.
//
// Public surface follows the reference (tensor.h:33-243) so that operator and model
// code reads the same; additions for this backend are Device::kHIP and the two
// Copy() branches that move data through the C ABI (frhip_memcpy).  The reference's
// msgpack-c dependency is replaced by the small reader in msgpack_lite.h.
#pragma once

#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <iosfwd>
#include <memory>
#include <optional>
#include <string>
#include <type_traits>
#include <vector>

#include "check.h"
#include "kernels/allocator.h"

namespace rwkv {

enum class DType { kUndefined, kInt4, kInt8, kFloat16, kFloat32, kInt32, kInt64 };

// kHIP is appended so that the numeric values of the reference's devices are unchanged
// (tensor.h:43-50).
enum class Device { kCPU, kCUDA, kNCNNMeta, kONNXMeta, kNCNN, kONNX, kHIP };

// IEEE binary16 storage type on the host.  Conversions are round-to-nearest-even.
struct float16 {
  uint16_t bits = 0;
  float16() = default;
  float16(float f);  // NOLINT: implicit, like half_float::half
  operator float() const;  // NOLINT
};

std::optional<Device> &default_dispatch_device();

template <typename T> inline const DType dtype_v = DType::kFloat32;
template <> inline const DType dtype_v<float16> = DType::kFloat16;
template <> inline const DType dtype_v<uint8_t> = DType::kInt8;
template <> inline const DType dtype_v<int8_t> = DType::kInt8;
template <> inline const DType dtype_v<int32_t> = DType::kInt32;
template <> inline const DType dtype_v<int64_t> = DType::kInt64;

using LengthType = int64_t;
using Shape = std::vector<LengthType>;

std::ostream &operator<<(std::ostream &os, const Shape &shape);
std::ostream &operator<<(std::ostream &os, DType dtype);
std::string dtype_to_string(DType dtype);
std::string shape_str(const Shape &shape);

inline LengthType num_elements(const Shape &shape) {
  LengthType n = 1;
  for (auto d : shape) n *= d;
  return n;
}

int32_t elem_size(DType dtype);

struct Range {
  int start, interval, end;
  Range(int start, int interval, int end) : start(start), interval(interval), end(end) {}
  static Range All;  // (0,0,0): the whole dimension
};

class TensorStorage {
public:
  TensorStorage(size_t nbytes, Device device);       // owns memory from allocator(device)
  TensorStorage(void *external_ptr, Device device);  // view: never frees
  // view into another storage, which it keeps alive
  TensorStorage(void *ptr_inside, std::shared_ptr<TensorStorage> owner);
  ~TensorStorage();
  void *data_ptr() const { return _data; }
  Device device() const { return _device; }
  size_t nbytes() const { return _nbytes; }
  FR_DISALLOW_COPY_AND_MOVE(TensorStorage);

private:
  void *_data = nullptr;
  size_t _nbytes = 0;
  bool _is_view = false;
  Device _device;
  std::shared_ptr<TensorStorage> _owner;
};

class Tensor {
public:
  Tensor() = default;
  template <typename T = void> const T *data_ptr() const {
    RV_CHECK((std::is_same_v<T, void> || dtype_v<T> == _dtype));
    return static_cast<const T *>(_storage->data_ptr());
  }
  template <typename T = void> T *data_ptr() {
    RV_CHECK((std::is_same_v<T, void> || dtype_v<T> == _dtype));
    return static_cast<T *>(_storage->data_ptr());
  }
  bool defined() const { return static_cast<bool>(_storage); }
  // Number of tensors (and sub-views) that share this tensor's storage, this one included.
  long storage_use_count() const { return _storage.use_count(); }
  bool shares_storage_with(const Tensor &other) const { return _storage && _storage == other._storage; }
  DType dtype() const { return _dtype; }
  Device device() const { return _storage->device(); }
  const Shape &sizes() const { return _shape; }
  const Shape &shape() const { return _shape; }
  LengthType size(int64_t dim) const { return _shape[dim < 0 ? dim + (int64_t)_shape.size() : dim]; }
  LengthType numel() const { return num_elements(_shape); }
  int32_t elem_size() const { return ::rwkv::elem_size(_dtype); }
  size_t nbytes() const { return static_cast<size_t>(numel()) * elem_size(); }

  Tensor view(const Shape &shape) const;
  Tensor reshape(const Shape &shape) const;
  Tensor flatten() const;
  Tensor unsqueeze(int dim) const;
  Tensor squeeze(int dim) const;
  Tensor slice(const std::vector<Range> &ranges) const;
  Tensor slice(const std::initializer_list<Range> &ranges) const;
  Tensor cat(const Tensor &other, int dim) const;
  Tensor transpose(int dim_a, int dim_b) const;

  static Tensor Empty(const Shape &shape, DType dtype, Device device);
  static Tensor FromPtr(void *ptr, const Shape &shape, DType dtype, Device device);
  static Tensor FromOther(const Tensor &other, const Shape &shape);
  // A tensor of `shape` (other's dtype) starting `byte_offset` bytes into `other`; shares its storage.
  static Tensor SubView(const Tensor &other, size_t byte_offset, const Shape &shape);

  std::string name;
  bool is_constant = false;

private:
  std::shared_ptr<TensorStorage> _storage;
  Shape _shape;
  DType _dtype = DType::kUndefined;
};

Tensor operator+(const Tensor &lhs, const Tensor &rhs);
Tensor operator-(const Tensor &lhs, const Tensor &rhs);
Tensor operator-(float lhs, const Tensor &rhs);
Tensor operator*(const Tensor &lhs, const Tensor &rhs);
Tensor operator/(const Tensor &lhs, const Tensor &rhs);

// Blocking copy between devices (reference: tensor.cpp:58-96).  CPU<->HIP and HIP->HIP
// go through frhip_memcpy; the copy is also the synchronisation point of a decode step.
Tensor Copy(const Tensor &x, Device device, bool always_copy = false);

void print_n(const Tensor &x, const std::string &name, int skip, int cnt = 20);

}  // namespace rwkv
