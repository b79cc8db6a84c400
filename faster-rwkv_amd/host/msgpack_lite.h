// A minimal MessagePack reader/writer: exactly what the `.fr` weight files
// (tools/convert_weight.py:12-55: maps, arrays, str, bin, ints, floats) and the state
// files (model.cpp:89-143) use.  Parsed values hold views into the input buffer for
// str/bin payloads, so the buffer must outlive them.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

#include "check.h"
#include "tensor.h"

namespace rwkv::mp {

struct Value {
  enum Kind { kNil, kBool, kInt, kFloat, kStr, kBin, kArray, kMap } kind = kNil;
  int64_t i = 0;
  double f = 0;
  std::string_view s;  // str or bin payload
  std::vector<Value> arr;
  std::vector<std::pair<Value, Value>> map;

  bool is_array() const { return kind == kArray; }
  bool is_map() const { return kind == kMap; }
  const Value *find(std::string_view key) const {
    for (const auto &kv : map)
      if (kv.first.kind == kStr && kv.first.s == key) return &kv.second;
    return nullptr;
  }
  const Value &at(std::string_view key) const {
    const Value *v = find(key);
    RV_CHECK(v != nullptr) << "msgpack: missing key " << std::string(key);
    return *v;
  }
  int64_t as_int() const {
    RV_CHECK(kind == kInt || kind == kFloat);
    return kind == kInt ? i : static_cast<int64_t>(f);
  }
  std::string as_str() const {
    RV_CHECK(kind == kStr || kind == kBin);
    return std::string(s);
  }
};

class Reader {
public:
  Reader(const char *p, size_t n) : _p(reinterpret_cast<const uint8_t *>(p)), _end(_p + n) {}
  Value next() {
    need(1);
    const uint8_t b = *_p++;
    Value v;
    if (b <= 0x7f) return integer(b);
    if (b >= 0xe0) return integer(static_cast<int8_t>(b));
    if ((b & 0xf0) == 0x80) return map(b & 0x0f);
    if ((b & 0xf0) == 0x90) return array(b & 0x0f);
    if ((b & 0xe0) == 0xa0) return blob(Value::kStr, b & 0x1f);
    switch (b) {
      case 0xc0: return v;
      case 0xc2: v.kind = Value::kBool; v.i = 0; return v;
      case 0xc3: v.kind = Value::kBool; v.i = 1; return v;
      case 0xc4: return blob(Value::kBin, be(1));
      case 0xc5: return blob(Value::kBin, be(2));
      case 0xc6: return blob(Value::kBin, be(4));
      case 0xca: { uint32_t u = static_cast<uint32_t>(be(4)); float f; std::memcpy(&f, &u, 4); v.kind = Value::kFloat; v.f = f; return v; }
      case 0xcb: { uint64_t u = be(8); double d; std::memcpy(&d, &u, 8); v.kind = Value::kFloat; v.f = d; return v; }
      case 0xcc: return integer(static_cast<int64_t>(be(1)));
      case 0xcd: return integer(static_cast<int64_t>(be(2)));
      case 0xce: return integer(static_cast<int64_t>(be(4)));
      case 0xcf: return integer(static_cast<int64_t>(be(8)));
      case 0xd0: return integer(static_cast<int8_t>(be(1)));
      case 0xd1: return integer(static_cast<int16_t>(be(2)));
      case 0xd2: return integer(static_cast<int32_t>(be(4)));
      case 0xd3: return integer(static_cast<int64_t>(be(8)));
      case 0xd9: return blob(Value::kStr, be(1));
      case 0xda: return blob(Value::kStr, be(2));
      case 0xdb: return blob(Value::kStr, be(4));
      case 0xdc: return array(be(2));
      case 0xdd: return array(be(4));
      case 0xde: return map(be(2));
      case 0xdf: return map(be(4));
      default: RV_UNIMPLEMENTED() << "msgpack: unsupported type byte " << static_cast<int>(b);
    }
  }
  bool done() const { return _p == _end; }

private:
  void need(size_t n) const { RV_CHECK(static_cast<size_t>(_end - _p) >= n) << "msgpack: truncated input"; }
  uint64_t be(int n) {
    need(static_cast<size_t>(n));
    uint64_t v = 0;
    for (int i = 0; i < n; i++) v = (v << 8) | *_p++;
    return v;
  }
  static Value integer(int64_t i) {
    Value v;
    v.kind = Value::kInt;
    v.i = i;
    return v;
  }
  Value blob(Value::Kind k, uint64_t n) {
    need(n);
    Value v;
    v.kind = k;
    v.s = std::string_view(reinterpret_cast<const char *>(_p), n);
    _p += n;
    return v;
  }
  Value array(uint64_t n) {
    Value v;
    v.kind = Value::kArray;
    v.arr.reserve(n);
    for (uint64_t i = 0; i < n; i++) v.arr.push_back(next());
    return v;
  }
  Value map(uint64_t n) {
    Value v;
    v.kind = Value::kMap;
    v.map.reserve(n);
    for (uint64_t i = 0; i < n; i++) {
      Value k = next();
      Value val = next();
      v.map.emplace_back(std::move(k), std::move(val));
    }
    return v;
  }
  const uint8_t *_p, *_end;
};

inline Value parse(const char *p, size_t n) { return Reader(p, n).next(); }

// {dtype: "torch.float16"|..., data: bin, shape: [..]} -> CPU tensor owning a copy
// (reference: Tensor::FromMsgPack, tensor.cpp:127-151).
inline Tensor to_tensor(const Value &v) {
  RV_CHECK(v.is_map());
  const std::string dt = v.at("dtype").as_str();
  DType dtype;
  if (dt == "torch.int8" || dt == "torch.uint8") dtype = DType::kInt8;
  else if (dt == "torch.float16") dtype = DType::kFloat16;
  else if (dt == "torch.float32") dtype = DType::kFloat32;
  else RV_UNIMPLEMENTED() << "msgpack tensor dtype " << dt;
  Shape shape;
  for (const auto &d : v.at("shape").arr) shape.push_back(d.as_int());
  const Value &data = v.at("data");
  RV_CHECK(data.kind == Value::kBin || data.kind == Value::kStr);
  Tensor t = Tensor::Empty(shape, dtype, Device::kCPU);
  RV_CHECK(data.s.size() == t.nbytes()) << "msgpack tensor: payload size does not match shape";
  std::memcpy(t.data_ptr(), data.s.data(), data.s.size());
  return t;
}

struct Writer {
  std::string buf;
  void byte(uint8_t b) { buf.push_back(static_cast<char>(b)); }
  void be(uint64_t v, int n) {
    for (int i = n - 1; i >= 0; i--) byte(static_cast<uint8_t>(v >> (8 * i)));
  }
  void array(size_t n) {
    if (n < 16) byte(static_cast<uint8_t>(0x90 | n));
    else if (n < 65536) { byte(0xdc); be(n, 2); }
    else { byte(0xdd); be(n, 4); }
  }
  void map(size_t n) {
    if (n < 16) byte(static_cast<uint8_t>(0x80 | n));
    else { byte(0xde); be(n, 2); }
  }
  void str(std::string_view s) {
    if (s.size() < 32) byte(static_cast<uint8_t>(0xa0 | s.size()));
    else if (s.size() < 256) { byte(0xd9); be(s.size(), 1); }
    else { byte(0xda); be(s.size(), 2); }
    buf.append(s);
  }
  void bin(const void *p, size_t n) {
    if (n < 256) { byte(0xc4); be(n, 1); }
    else if (n < 65536) { byte(0xc5); be(n, 2); }
    else { byte(0xc6); be(n, 4); }
    buf.append(static_cast<const char *>(p), n);
  }
  void integer(int64_t v) {
    if (v >= 0 && v < 128) byte(static_cast<uint8_t>(v));
    else if (v >= 0) { byte(0xcf); be(static_cast<uint64_t>(v), 8); }
    else { byte(0xd3); be(static_cast<uint64_t>(v), 8); }
  }
};

}  // namespace rwkv::mp
