#include "tensor.h"

#include <algorithm>
#include <cmath>
#include <iomanip>
#include <iostream>

#include "frhip.h"
#include "kernels/kernels.h"

namespace rwkv {

Range Range::All = Range(0, 0, 0);

// ---- binary16 <-> binary32, round to nearest even -----------------------------
float16::float16(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) {  // inf / nan
    bits = static_cast<uint16_t>(sign | 0x7C00u | (absx > 0x7F800000u ? 0x200u : 0u));
    return;
  }
  if (absx >= 0x477FF000u) {  // rounds to >= 65520 -> inf
    bits = static_cast<uint16_t>(sign | 0x7C00u);
    return;
  }
  if (absx < 0x33000001u) {  // <= 2^-25: rounds to zero
    bits = static_cast<uint16_t>(sign);
    return;
  }
  const int e = static_cast<int>(absx >> 23) - 127;
  uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;  // 24-bit significand
  const int shift = (e >= -14) ? 13 : 13 + (-14 - e);
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  if (e >= -14)
    bits = static_cast<uint16_t>(sign | ((static_cast<uint32_t>(e + 14) << 10) + q));
  else
    bits = static_cast<uint16_t>(sign | q);
}

float16::operator float() const {
  const uint32_t sign = (static_cast<uint32_t>(bits) & 0x8000u) << 16;
  const uint32_t exp = (bits >> 10) & 0x1Fu;
  uint32_t man = bits & 0x3FFu;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) {
      x = sign;
    } else {
      int sh = 0;
      while (!(man & 0x400u)) {
        man <<= 1;
        sh++;
      }
      x = sign | (static_cast<uint32_t>(113 - sh) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    x = sign | 0x7F800000u | (man << 13);
  } else {
    x = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}

std::optional<Device> &default_dispatch_device() {
  static std::optional<Device> d = std::nullopt;
  return d;
}

std::string dtype_to_string(DType dtype) {
  switch (dtype) {
    case DType::kFloat32: return "fp32";
    case DType::kFloat16: return "fp16";
    case DType::kInt32: return "int32";
    case DType::kInt64: return "int64";
    case DType::kInt8: return "int8";
    case DType::kInt4: return "int4";
    default: RV_UNIMPLEMENTED();
  }
}

int32_t elem_size(DType dtype) {
  switch (dtype) {
    case DType::kInt8: return 1;
    case DType::kFloat16: return 2;
    case DType::kFloat32: return 4;
    case DType::kInt32: return 4;
    case DType::kInt64: return 8;
    default: RV_UNIMPLEMENTED() << "Unsupported dtype";
  }
}

std::ostream &operator<<(std::ostream &os, const Shape &shape) {
  os << "(";
  for (size_t i = 0; i < shape.size(); i++) os << shape[i] << (i + 1 < shape.size() ? ", " : "");
  return os << ")";
}

std::string shape_str(const Shape &shape) {
  std::ostringstream os;
  os << shape;
  return os.str();
}

std::ostream &operator<<(std::ostream &os, DType dtype) { return os << dtype_to_string(dtype); }

// ---- storage -------------------------------------------------------------------
TensorStorage::TensorStorage(size_t nbytes, Device device) : _nbytes(nbytes), _is_view(false), _device(device) {
  _data = allocator(device).Allocate(nbytes);
}

TensorStorage::TensorStorage(void *external_ptr, Device device)
    : _data(external_ptr), _nbytes(0), _is_view(true), _device(device) {}

TensorStorage::TensorStorage(void *ptr_inside, std::shared_ptr<TensorStorage> owner)
    : _data(ptr_inside), _nbytes(0), _is_view(true), _device(owner->device()), _owner(std::move(owner)) {}

TensorStorage::~TensorStorage() {
  if (!_is_view && _data) allocator(_device).Deallocate(_data);
}

namespace {
std::string next_name() {
  static int id = 0;
  return "tensor_" + std::to_string(id++);
}
}  // namespace

Tensor Tensor::Empty(const Shape &shape, DType dtype, Device device) {
  Tensor t;
  t._storage = std::make_shared<TensorStorage>(static_cast<size_t>(num_elements(shape)) * ::rwkv::elem_size(dtype), device);
  t._shape = shape;
  t._dtype = dtype;
  t.name = next_name();
  return t;
}

Tensor Tensor::FromPtr(void *ptr, const Shape &shape, DType dtype, Device device) {
  Tensor t;
  t._storage = std::make_shared<TensorStorage>(ptr, device);
  t._shape = shape;
  t._dtype = dtype;
  t.name = next_name();
  return t;
}

Tensor Tensor::FromOther(const Tensor &other, const Shape &shape) {
  Tensor t;
  t._storage = other._storage;
  t._shape = shape;
  t._dtype = other._dtype;
  t.name = next_name();
  return t;
}

Tensor Tensor::SubView(const Tensor &other, size_t byte_offset, const Shape &shape) {
  RV_CHECK(other.defined());
  RV_CHECK(byte_offset + static_cast<size_t>(num_elements(shape)) * other.elem_size() <= other.nbytes())
      << "SubView: range runs past the source tensor";
  Tensor t;
  t._storage = std::make_shared<TensorStorage>(static_cast<char *>(other._storage->data_ptr()) + byte_offset, other._storage);
  t._shape = shape;
  t._dtype = other._dtype;
  t.name = next_name();
  return t;
}

Tensor Tensor::view(const Shape &shape) const { return ::rwkv::reshape(*this, shape); }
Tensor Tensor::reshape(const Shape &shape) const { return ::rwkv::reshape(*this, shape); }
Tensor Tensor::flatten() const { return ::rwkv::flatten(*this); }
Tensor Tensor::unsqueeze(int dim) const { return ::rwkv::unsqueeze(*this, dim); }
Tensor Tensor::squeeze(int dim) const { return ::rwkv::squeeze(*this, dim); }
Tensor Tensor::slice(const std::vector<Range> &ranges) const { return ::rwkv::slice(*this, ranges); }
Tensor Tensor::slice(const std::initializer_list<Range> &ranges) const {
  return ::rwkv::slice(*this, std::vector<Range>(ranges));
}
Tensor Tensor::cat(const Tensor &other, int dim) const { return ::rwkv::cat(*this, other, dim); }
Tensor Tensor::transpose(int a, int b) const { return ::rwkv::transpose(*this, a, b); }

Tensor operator+(const Tensor &l, const Tensor &r) { return add(l, r); }
Tensor operator-(const Tensor &l, const Tensor &r) { return sub(l, r); }
Tensor operator-(float l, const Tensor &r) { return sub(l, r); }
Tensor operator*(const Tensor &l, const Tensor &r) { return mul(l, r); }
Tensor operator/(const Tensor &l, const Tensor &r) { return div(l, r); }

Tensor Copy(const Tensor &x, Device device, bool always_copy) {
  if (x.device() == device && !always_copy) return x;
  Tensor y = Tensor::Empty(x.sizes(), x.dtype(), device);
  y.name = x.name;
  const size_t n = x.nbytes();
  const Device src = x.device();
  if (src == Device::kCPU && device == Device::kCPU) {
    std::memcpy(y.data_ptr(), x.data_ptr(), n);
  } else if (src == Device::kHIP && device == Device::kCPU) {
    FRHIP_CHECK(frhip_memcpy(y.data_ptr(), x.data_ptr(), n, FRHIP_D2H));
  } else if (src == Device::kCPU && device == Device::kHIP) {
    FRHIP_CHECK(frhip_memcpy(y.data_ptr(), x.data_ptr(), n, FRHIP_H2D));
  } else if (src == Device::kHIP && device == Device::kHIP) {
    FRHIP_CHECK(frhip_memcpy(y.data_ptr(), x.data_ptr(), n, FRHIP_D2D));
  } else {
    RV_UNIMPLEMENTED() << "Copy from device " << static_cast<int>(src) << " to device " << static_cast<int>(device)
                       << " is not supported yet.";
  }
  return y;
}

void print_n(const Tensor &x, const std::string &name, int skip, int cnt) {
  Tensor c = Copy(x, Device::kCPU);
  const int n = static_cast<int>(x.numel());
  if (cnt > n) {
    cnt = n;
    skip = 0;
  }
  std::cout << ">>>>>>>> " << name << ": " << std::fixed << std::setprecision(6);
  for (int i = 0; i < cnt; i++) {
    if (x.dtype() == DType::kFloat32)
      std::cout << c.data_ptr<float>()[skip + i] << ", ";
    else if (x.dtype() == DType::kFloat16)
      std::cout << static_cast<float>(c.data_ptr<float16>()[skip + i]) << ", ";
  }
  std::cout << std::endl;
}

// ---- registry --------------------------------------------------------------------
KernelRegistry &KernelRegistry::Instance() {
  static KernelRegistry r;
  return r;
}

void KernelRegistry::Register(const std::string &name, Device device, std::any kernel, int /*priority*/) {
  _table[{name, device}] = std::move(kernel);
}

bool KernelRegistry::Has(const std::string &name, Device device) const {
  return _table.find({name, device}) != _table.end();
}

}  // namespace rwkv
