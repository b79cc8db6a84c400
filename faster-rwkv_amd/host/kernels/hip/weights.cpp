// Packed weights of the `hip` backend and the host-side uint8 quantiser.
#include <algorithm>
#include <cmath>
#include <functional>
#include <cstring>
#include <mutex>
#include <thread>
#include <unordered_map>

#include "kernels/hip/context.h"
#include "kernels/kernels.h"

namespace rwkv {
namespace hip {

frhip_stream stream() {
  static frhip_stream s = []() {
    int n = 0;
    FRHIP_CHECK(frhip_device_count(&n));
    const char *dev = std::getenv("FR_HIP_DEVICE");
    FRHIP_CHECK(frhip_init(dev ? std::atoi(dev) : 0));
    frhip_stream st = nullptr;
    FRHIP_CHECK(frhip_stream_create(&st));
    return st;
  }();
  return s;
}

namespace {
std::mutex g_mu;
std::unordered_map<const void *, std::shared_ptr<PackedWeight>> &table() {
  static auto *t = new std::unordered_map<const void *, std::shared_ptr<PackedWeight>>();
  return *t;
}
}  // namespace

void register_weight(const void *p, std::shared_ptr<PackedWeight> w) {
  std::lock_guard<std::mutex> lock(g_mu);
  table()[p] = std::move(w);
}

void unregister_weight(const void *p) {
  std::lock_guard<std::mutex> lock(g_mu);
  table().erase(p);
}

const frhip_weight *find_weight(const Tensor &t) {
  if (!t.defined() || t.device() != Device::kHIP) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = table().find(t.data_ptr());
  return it == table().end() ? nullptr : &it->second->desc;
}

// FR_HIP_SEQ_IMAGE=1 keeps the images (read per call, like FR_HIP_GENERIC).  Unset or 0: never -- a caller who chose
// uint8 weights chose their footprint, and the images would triple it (2 more bytes per weight: a 14B model goes from
// 14 to 42 GB).  On a 288 GB part that is often the trade to take (no expansion per prompt), so it is one switch away.
static bool keep_images() {
  const char *e = std::getenv("FR_HIP_SEQ_IMAGE");
  return e != nullptr && std::atoi(e) != 0;
}

const frhip_weight *find_seq_weight(const Tensor &t, int rows) {
  if (rows < FRHIP_SEQ_EXPAND_ROWS || !keep_images()) return find_weight(t);
  if (!t.defined() || t.device() != Device::kHIP) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = table().find(t.data_ptr());
  if (it == table().end()) return nullptr;
  PackedWeight &w = *it->second;
  if (w.desc.dtype != FRHIP_U8 || w.no_image) return &w.desc;
  if (!w.image.defined()) {
    Tensor img;
    try {
      img = Tensor::Empty({static_cast<LengthType>(w.desc.N), static_cast<LengthType>(w.desc.K)}, DType::kFloat16,
                          Device::kHIP);
    } catch (const std::exception &) {  // no room: this weight is expanded per call, as without images
      w.no_image = true;
      return &w.desc;
    }
    // on the backend's stream, like every product that will read it
    FRHIP_CHECK(frhip_dequant_u8(&w.desc, img.data_ptr(), stream()));
    w.image = img;
    w.image_desc = frhip_weight{};
    w.image_desc.data = w.image.data_ptr();
    w.image_desc.K = w.desc.K;
    w.image_desc.N = w.desc.N;
    w.image_desc.dtype = FRHIP_F16;
  }
  return &w.image_desc;
}

static inline float h2f(uint16_t b) {
  float16 h;
  h.bits = b;
  return static_cast<float>(h);
}
static inline uint16_t f2h(float f) { return float16(f).bits; }

static void parallel_for(int n, const std::function<void(int, int)> &fn) {
  int nt = static_cast<int>(std::thread::hardware_concurrency());
  nt = std::max(1, std::min(nt, 16));
  if (n < 64) nt = 1;
  std::vector<std::thread> th;
  for (int t = 0; t < nt; t++) {
    int lo = static_cast<int>((long long)n * t / nt), hi = static_cast<int>((long long)n * (t + 1) / nt);
    th.emplace_back([=, &fn]() { fn(lo, hi); });
  }
  for (auto &t : th) t.join();
}

void quantize_u8(const uint16_t *w, int K, int N, uint8_t *q, uint16_t *mx, uint16_t *rx, uint16_t *my,
                 uint16_t *ry) {
  std::vector<float> r(static_cast<size_t>(K) * N);
  // mx[n] = min over k
  std::vector<float> mxf(N), rxf(N), myf(K), ryf(K);
  parallel_for(N, [&](int lo, int hi) {
    for (int n = lo; n < hi; n++) {
      float m = h2f(w[n]);
      for (int k = 1; k < K; k++) m = std::min(m, h2f(w[(size_t)k * N + n]));
      mx[n] = f2h(m);
      mxf[n] = h2f(mx[n]);
    }
  });
  // r = w - mx ; my[k] = min over n ; r -= my
  parallel_for(K, [&](int lo, int hi) {
    for (int k = lo; k < hi; k++) {
      float *rk = r.data() + (size_t)k * N;
      float m = INFINITY;
      for (int n = 0; n < N; n++) {
        rk[n] = h2f(w[(size_t)k * N + n]) - mxf[n];
        m = std::min(m, rk[n]);
      }
      my[k] = f2h(m);
      myf[k] = h2f(my[k]);
      for (int n = 0; n < N; n++) rk[n] = rk[n] - myf[k];
    }
  });
  // rx[n] = max over k (floored so that a constant column does not divide by zero) ; r /= rx
  parallel_for(N, [&](int lo, int hi) {
    for (int n = lo; n < hi; n++) {
      float m = -INFINITY;
      for (int k = 0; k < K; k++) m = std::max(m, r[(size_t)k * N + n]);
      rx[n] = f2h(std::max(m, 1e-4f));
      rxf[n] = h2f(rx[n]);
    }
  });
  parallel_for(K, [&](int lo, int hi) {
    for (int k = lo; k < hi; k++) {
      float *rk = r.data() + (size_t)k * N;
      float m = -INFINITY;
      for (int n = 0; n < N; n++) {
        rk[n] = rk[n] / rxf[n];
        m = std::max(m, rk[n]);
      }
      ry[k] = f2h(std::max(m, 1e-4f));
      ryf[k] = h2f(ry[k]);
      for (int n = 0; n < N; n++) {
        float v = std::nearbyintf((rk[n] / ryf[k]) * 255.0f);
        q[(size_t)k * N + n] = static_cast<uint8_t>(std::min(255.0f, std::max(0.0f, v)));
      }
    }
  });
}

static Tensor upload(const void *host, size_t bytes, const Shape &shape, DType dtype) {
  Tensor t = Tensor::Empty(shape, dtype, Device::kHIP);
  FRHIP_CHECK(frhip_memcpy(t.data_ptr(), host, bytes, FRHIP_H2D));
  return t;
}

static Tensor finish(std::shared_ptr<PackedWeight> pw, int K, int N, DType dtype, const std::string &name) {
  Tensor view = Tensor::FromPtr(const_cast<void *>(pw->desc.data), {K, N}, dtype, Device::kHIP);
  view.name = name;
  view.is_constant = true;
  register_weight(pw->desc.data, pw);
  return view;
}

static Tensor pack_matrix(const void *host_kn, int K, int N, int elem) {
  const size_t bytes = static_cast<size_t>(K) * N * elem;
  const DType dt = elem == 2 ? DType::kFloat16 : DType::kInt8;
  Tensor staged = upload(host_kn, bytes, {K, N}, dt);
  Tensor packed = Tensor::Empty({N, K}, dt, Device::kHIP);
  FRHIP_CHECK(frhip_pack_transpose(staged.data_ptr(), packed.data_ptr(), K, N, elem, stream()));
  FRHIP_CHECK(frhip_stream_sync(stream()));
  return packed;
}

Tensor make_weight_from_host_u8(const uint8_t *q, const void *mx, const void *rx, const void *my, const void *ry,
                                int K, int N, const std::string &name) {
  RV_CHECK(K % 16 == 0) << "hip int8 weights need the input dimension to be a multiple of 16, got " << K;
  auto pw = std::make_shared<PackedWeight>();
  pw->owners.push_back(pack_matrix(q, K, N, 1));
  pw->owners.push_back(upload(mx, 2 * (size_t)N, {N}, DType::kFloat16));
  pw->owners.push_back(upload(rx, 2 * (size_t)N, {N}, DType::kFloat16));
  pw->owners.push_back(upload(my, 2 * (size_t)K, {K}, DType::kFloat16));
  pw->owners.push_back(upload(ry, 2 * (size_t)K, {K}, DType::kFloat16));
  pw->desc.data = pw->owners[0].data_ptr();
  pw->desc.mx = pw->owners[1].data_ptr();
  pw->desc.rx = pw->owners[2].data_ptr();
  pw->desc.my = pw->owners[3].data_ptr();
  pw->desc.ry = pw->owners[4].data_ptr();
  pw->desc.K = K;
  pw->desc.N = N;
  pw->desc.dtype = FRHIP_U8;
  return finish(pw, K, N, DType::kInt8, name);
}

Tensor make_weight_from_host(const void *src_kn, int K, int N, DType dtype, const std::string &name) {
  RV_CHECK(K % 16 == 0) << "hip weights need the input dimension to be a multiple of 16, got " << K;
  if (dtype == DType::kInt8) {
    std::vector<uint8_t> q(static_cast<size_t>(K) * N);
    std::vector<uint16_t> mx(N), rx(N), my(K), ry(K);
    quantize_u8(static_cast<const uint16_t *>(src_kn), K, N, q.data(), mx.data(), rx.data(), my.data(), ry.data());
    return make_weight_from_host_u8(q.data(), mx.data(), rx.data(), my.data(), ry.data(), K, N, name);
  }
  RV_CHECK(dtype == DType::kFloat16);
  auto pw = std::make_shared<PackedWeight>();
  pw->owners.push_back(pack_matrix(src_kn, K, N, 2));
  pw->desc.data = pw->owners[0].data_ptr();
  pw->desc.K = K;
  pw->desc.N = N;
  pw->desc.dtype = FRHIP_F16;
  return finish(pw, K, N, DType::kFloat16, name);
}

}  // namespace hip
}  // namespace rwkv
