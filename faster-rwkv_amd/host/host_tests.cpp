// Unit tests of the host layer that need no GPU: run by tests/test_host_cpu.py.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>

#include "kernels/kernels.h"
#include "model.h"
#include "msgpack_lite.h"

using namespace rwkv;

static int g_fail = 0;
#define EXPECT(cond)                                                   \
  do {                                                                 \
    if (!(cond)) {                                                     \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);    \
      g_fail++;                                                        \
    }                                                                  \
  } while (0)

template <typename F> static std::string thrown(F &&f) {
  try {
    f();
  } catch (const std::exception &e) {
    return e.what();
  }
  return "";
}

static void test_float16() {
  struct { float f; uint16_t h; } kv[] = {
      {0.f, 0x0000}, {1.f, 0x3C00}, {-2.f, 0xC000}, {0.5f, 0x3800}, {65504.f, 0x7BFF}, {65520.f, 0x7C00},
      {65519.f, 0x7BFF}, {5.9604645e-8f, 0x0001}, {2.9802322e-8f, 0x0000}, {2.9802326e-8f, 0x0001},
      {6.1035156e-5f, 0x0400}, {0.1f, 0x2E66}, {1.0009765625f, 0x3C01}, {1.00048828125f, 0x3C00},
      {1.00146484375f, 0x3C02}, {-1e30f, 0xFC00}};
  for (auto &c : kv) EXPECT(float16(c.f).bits == c.h);
  for (uint32_t b = 0; b < 0x7C00; b++) {  // every finite half survives a round trip
    float16 h;
    h.bits = static_cast<uint16_t>(b);
    EXPECT(float16(static_cast<float>(h)).bits == b);
  }
  float16 inf;
  inf.bits = 0x7C00;
  EXPECT(std::isinf(static_cast<float>(inf)));
}

static void test_registry_and_ops() {
  // unknown kernel: std::runtime_error("kernel <name> not found"), as kernels/registry.h:21-23
  Tensor t = Tensor::Empty({4}, DType::kFloat32, Device::kCPU);
  EXPECT(thrown([&]() { layernorm(t, t, t); }) == "kernel layernorm not found");
  EXPECT(KernelRegistry::Instance().Has("att", Device::kHIP));
  EXPECT(KernelRegistry::Instance().Has("ffn", Device::kHIP));
  EXPECT(KernelRegistry::Instance().Has("model_forward", Device::kHIP));
  EXPECT(KernelRegistry::Instance().Has("allocator", Device::kHIP));
  EXPECT(!KernelRegistry::Instance().Has("att", Device::kCPU));
  // asking with the wrong pointer type is a bad_any_cast
  bool bad = false;
  try {
    KernelRegistry::Instance().Get<int (*)()>("fill_", Device::kCPU);
  } catch (const std::bad_any_cast &) {
    bad = true;
  }
  EXPECT(bad);
  // last registration wins
  static auto f1 = +[]() -> int { return 1; };
  static auto f2 = +[]() -> int { return 2; };
  KernelRegister r1("unit_test_op", Device::kCPU, f1), r2("unit_test_op", Device::kCPU, f2);
  EXPECT(KernelRegistry::Instance().Get<int (*)()>("unit_test_op", Device::kCPU)() == 2);

  // tests/test_ops.cpp:9-16 on the CPU side: fill, cast
  Tensor h = Tensor::Empty({256}, DType::kFloat16, Device::kCPU);
  fill_(h, 1.0f);
  Tensor f = cast_dtype(h, DType::kFloat32);
  EXPECT(f.data_ptr<float>()[255] == 1.0f);
  EXPECT(reinterpret_cast<uintptr_t>(h.data_ptr()) % 512 == 0);  // allocator.h: 512-byte alignment

  // reshape: views share storage, -1 is inferred, bad shapes throw
  Tensor v = f.reshape({-1, 64});
  EXPECT(v.size(0) == 4 && v.size(1) == 64 && v.data_ptr() == f.data_ptr());
  EXPECT(!thrown([&]() { f.reshape({7, -1}); }).empty());
  EXPECT(!thrown([&]() { f.reshape({-1, -1}); }).empty());
  EXPECT(unsqueeze(f, 0).shape() == Shape({1, 256}));
  EXPECT(squeeze(unsqueeze(f, 0), 0).shape() == Shape({256}));
  EXPECT(flatten(v).shape() == Shape({256}));
  // dtype-checked access (tensor.h:142-145)
  EXPECT(!thrown([&]() { f.data_ptr<float16>(); }).empty());
  // Copy on the same device returns the same storage unless always_copy
  EXPECT(Copy(f, Device::kCPU).data_ptr() == f.data_ptr());
  EXPECT(Copy(f, Device::kCPU, true).data_ptr() != f.data_ptr());
}

static void test_errors() {
  std::string m = thrown([]() { RV_CHECK(1 == 2) << "ctx " << 7; });
  EXPECT(m.find("Check \"1 == 2\" failed") != std::string::npos && m.find("ctx 7") != std::string::npos);
  EXPECT(thrown([]() { RV_UNIMPLEMENTED() << "x"; }).find("Unimplemented") != std::string::npos);
  EXPECT(thrown([]() { Model m("nothing.fr", "tpu fp16"); }).find("unknown device") != std::string::npos);
  EXPECT(thrown([]() { Model m("nothing.fr", "hip"); }).find("unknown dtype") != std::string::npos);
  int evaluated = 0;
  RV_CHECK(++evaluated == 1);
  EXPECT(evaluated == 1);  // the condition is evaluated once when it holds
}

static void test_msgpack() {
  mp::Writer w;
  w.map(3);
  w.str("n_layer");
  w.integer(24);
  w.str("neg");
  w.integer(-5);
  w.str("t");
  w.map(3);
  w.str("dtype");
  w.str("torch.float16");
  const uint16_t payload[6] = {0x3C00, 0x4000, 0x4200, 0x4400, 0x4500, 0x4600};
  w.str("data");
  w.bin(payload, sizeof(payload));
  w.str("shape");
  w.array(2);
  w.integer(2);
  w.integer(3);
  mp::Value v = mp::parse(w.buf.data(), w.buf.size());
  EXPECT(v.is_map() && v.at("n_layer").as_int() == 24 && v.at("neg").as_int() == -5);
  Tensor t = mp::to_tensor(v.at("t"));
  EXPECT(t.shape() == Shape({2, 3}) && t.dtype() == DType::kFloat16);
  EXPECT(static_cast<float>(t.data_ptr<float16>()[5]) == 6.0f);
  EXPECT(!thrown([&]() { mp::parse(w.buf.data(), w.buf.size() - 3); }).empty());  // truncated
  EXPECT(!thrown([&]() { v.at("missing"); }).empty());
  // big containers and long strings use the 16/32-bit headers
  mp::Writer big;
  big.array(70000);
  for (int i = 0; i < 70000; i++) big.integer(i * 1000003LL);
  mp::Value bv = mp::parse(big.buf.data(), big.buf.size());
  EXPECT(bv.arr.size() == 70000 && bv.arr[69999].as_int() == 69999 * 1000003LL);
}

int main() {
  test_float16();
  test_registry_and_ops();
  test_errors();
  test_msgpack();
  if (g_fail == 0) std::printf("all host tests passed\n");
  return g_fail == 0 ? 0 : 1;
}
