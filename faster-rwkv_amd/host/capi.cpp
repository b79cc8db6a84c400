// A small C API over rwkv::Model for scripts and benchmarks (ctypes).  It adds nothing to
// the model; it only lets a non-C++ caller construct a Model with a strategy string, run
// it, and read the logits -- what chat.cpp / bench_model.cpp do in the reference.
#include <chrono>
#include <cmath>
#include <cstring>
#include <map>
#include <string>

#include "kernels/hip/context.h"
#include "kernels/hip/hip_model.h"
#include "kernels/kernels.h"
#include "model.h"
#include "sampler.h"

namespace rwkv::hip {
void allocator_stats(size_t *reserved, size_t *in_use, size_t *driver_calls);
size_t allocator_trim();
}

namespace {
thread_local std::string g_err;
template <typename F> auto guarded(F &&f) -> decltype(f()) {
  try {
    return f();
  } catch (const std::exception &e) {
    g_err = e.what();
    return -1;
  }
}
// First index of the maximum (Sampler::Sample with top_k = 1).  Two passes so that the
// compiler can vectorise the first: eight independent running maxima, then a scan for the value.
int argmax(const float *x, int n) {
  float m[8];
  for (int j = 0; j < 8; j++) m[j] = -INFINITY;
  int i = 0;
  for (; i + 8 <= n; i += 8)
    for (int j = 0; j < 8; j++) m[j] = x[i + j] > m[j] ? x[i + j] : m[j];
  float best = m[0];
  for (int j = 1; j < 8; j++) best = m[j] > best ? m[j] : best;
  for (; i < n; i++) best = x[i] > best ? x[i] : best;
  for (i = 0; i < n; i++)
    if (x[i] == best) return i;
  return 0;
}
}  // namespace

extern "C" {

const char *fr_last_error(void) { return g_err.c_str(); }

void *fr_model_create(const char *path, const char *strategy) {
  void *m = nullptr;
  guarded([&]() {
    m = new rwkv::Model(path, strategy);
    return 0;
  });
  return m;
}

void fr_model_free(void *m) { delete static_cast<rwkv::Model *>(m); }

// out[0..5] = n_layer, n_embd, n_att, n_ffn, n_head, vocab
int fr_model_info(void *m, int *out) {
  return guarded([&]() {
    auto *model = static_cast<rwkv::Model *>(m);
    out[0] = model->n_layer();
    out[1] = model->n_embd();
    out[2] = model->n_att();
    out[3] = model->n_ffn();
    out[4] = model->head_size();
    out[5] = static_cast<int>(model->_embd_weights.size());
    return 0;
  });
}

// Model::Run(ids): n == 1 one-token forward, n > 1 seq mode.  Returns the number of logits.
int fr_model_run(void *m, const int *ids, int n, float *logits, int capacity) {
  return guarded([&]() {
    auto *model = static_cast<rwkv::Model *>(m);
    rwkv::Tensor out = n == 1 ? model->Run(ids[0]) : model->Run(std::vector<int>(ids, ids + n));
    const int v = static_cast<int>(out.numel());
    if (v > capacity) throw FRException("logits buffer too small");
    std::memcpy(logits, out.data_ptr<float>(), sizeof(float) * static_cast<size_t>(v));
    return v;
  });
}

// ModelForwardSeq(model, device, ids, /*full_output=*/true) (kernels/kernels.h:279-284):
// logits of every position, [n][vocab] row-major.  Returns the number of floats written.
long long fr_model_run_full(void *m, const int *ids, int n, float *logits, long long capacity) {
  return guarded([&]() -> long long {
    auto *model = static_cast<rwkv::Model *>(m);
    rwkv::Tensor out = rwkv::Copy(
        rwkv::ModelForwardSeq(model, model->_act_device, std::vector<int>(ids, ids + n), true), rwkv::Device::kCPU);
    const long long v = static_cast<long long>(out.numel());
    if (v > capacity) throw FRException("logits buffer too small");
    std::memcpy(logits, out.data_ptr<float>(), sizeof(float) * static_cast<size_t>(v));
    return v;
  });
}

// Sampler (sampler.h:8-16).
void *fr_sampler_create(int seed, int seeded) {
  void *out = nullptr;
  guarded([&]() {
    auto *s = new rwkv::Sampler();
    if (seeded) s->set_seed(seed);
    out = s;
    return 0;
  });
  return out;
}

void fr_sampler_free(void *s) { delete static_cast<rwkv::Sampler *>(s); }

int fr_sampler_set_seed(void *s, int seed) {
  return guarded([&]() {
    static_cast<rwkv::Sampler *>(s)->set_seed(seed);
    return 0;
  });
}

// Sampler::Sample on a host buffer of n fp32 logits; returns the token id.
int fr_sampler_sample(void *s, const float *logits, int n, float temperature, int top_k, float top_p) {
  return guarded([&]() { return static_cast<rwkv::Sampler *>(s)->Sample(logits, n, temperature, top_k, top_p); });
}

// The generation loop of chat.cpp:56-92: feed first_id, adjust the host logits by the repetition
// penalties, sample, feed the sample, `steps` times.  As there, every token drawn so far has
// `frequency_penalty * count + presence_penalty` subtracted from its logit before the draw, in the order of the
// occurrence map, and its count is then multiplied by `penalty_decay` (chat.cpp:57-62); the drawn token's
// count goes up by one (chat.cpp:77).  The reference's values are 0.8, 0.8 and 0.996 (chat.cpp:22-24).  The
// adjustments its question-and-answer mode makes to two token ids of its own vocabulary (chat.cpp:63-74) belong
// to that front end and are not made here.  Returns the elapsed microseconds, or -1.
long long fr_chat_decode(void *m, void *sampler, int first_id, int steps, float temperature, int top_k, float top_p,
                         float presence_penalty, float frequency_penalty, float penalty_decay, int *out_ids) {
  return guarded([&]() -> long long {
    auto *model = static_cast<rwkv::Model *>(m);
    auto *smp = static_cast<rwkv::Sampler *>(sampler);
    std::map<int, float> occurrences;
    int id = first_id;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; i++) {
      // the logits are adjusted in place: Run's result is the caller's to change until the next-but-one call
      rwkv::Tensor out = rwkv::Copy(model->Run(id), rwkv::Device::kCPU);
      float *logits = out.data_ptr<float>();
      for (auto &[tok, count] : occurrences) {
        logits[tok] -= frequency_penalty * count + presence_penalty;
        count *= penalty_decay;
      }
      id = smp->Sample(out, temperature, top_k, top_p);
      occurrences[id]++;
      out_ids[i] = id;
    }
    return std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count();
  });
}

// The same loop without penalties.
long long fr_sample_decode(void *m, void *sampler, int first_id, int steps, float temperature, int top_k,
                           float top_p, int *out_ids) {
  return guarded([&]() -> long long {
    auto *model = static_cast<rwkv::Model *>(m);
    auto *smp = static_cast<rwkv::Sampler *>(sampler);
    int id = first_id;
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; i++) {
      rwkv::Tensor out = model->Run(id);
      id = smp->Sample(out, temperature, top_k, top_p);
      out_ids[i] = id;
    }
    return std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count();
  });
}

int fr_model_reset(void *m) {
  return guarded([&]() {
    static_cast<rwkv::Model *>(m)->ResetStates();
    return 0;
  });
}

int fr_model_save_state(void *m, const char *path) {
  return guarded([&]() {
    static_cast<rwkv::Model *>(m)->SaveStateFile(path);
    return 0;
  });
}

int fr_model_load_state(void *m, const char *path) {
  return guarded([&]() {
    static_cast<rwkv::Model *>(m)->LoadStateFile(path);
    return 0;
  });
}

// A snapshot as a C++ caller takes one: a copy of Model::states() (tensors that share storage with the
// model's, no device copy), to be handed back through set_states() later.
void *fr_model_snapshot(void *m) {
  void *out = nullptr;
  guarded([&]() {
    out = new rwkv::States(static_cast<rwkv::Model *>(m)->states());
    return 0;
  });
  return out;
}

int fr_model_restore(void *m, void *snapshot) {
  return guarded([&]() {
    static_cast<rwkv::Model *>(m)->set_states(*static_cast<rwkv::States *>(snapshot));
    return 0;
  });
}

void fr_snapshot_free(void *snapshot) { delete static_cast<rwkv::States *>(snapshot); }

// Copy state tensor (layer, index) to the host as raw bytes; returns its size in bytes.
int fr_model_get_state(void *m, int layer, int index, void *out, int capacity) {
  return guarded([&]() {
    auto *model = static_cast<rwkv::Model *>(m);
    rwkv::Tensor c = rwkv::Copy(model->states().at(layer).at(index), rwkv::Device::kCPU);
    const int n = static_cast<int>(c.nbytes());
    if (n > capacity) throw FRException("state buffer too small");
    std::memcpy(out, c.data_ptr(), static_cast<size_t>(n));
    return n;
  });
}

// Replace state tensor (layer, index) by `nbytes` raw bytes from the host (same shape and dtype), as
// LoadStateFile does for every tensor of a file (model.cpp:117-143).
int fr_model_set_state(void *m, int layer, int index, const void *data, int nbytes) {
  return guarded([&]() {
    auto *model = static_cast<rwkv::Model *>(m);
    rwkv::Tensor &dst = model->states().at(layer).at(index);
    if (static_cast<size_t>(nbytes) != dst.nbytes()) throw FRException("state tensor size mismatch");
    rwkv::Tensor t = rwkv::Tensor::Empty(dst.shape(), dst.dtype(), rwkv::Device::kCPU);
    std::memcpy(t.data_ptr(), data, static_cast<size_t>(nbytes));
    dst = rwkv::Copy(t, dst.device());
    return 0;
  });
}

// Greedy decoding as chat.cpp:56-92 does with top_k = 1: feed `first_id`, take the argmax of
// the returned (host) logits, feed it back.  out_ids receives `steps` tokens.  Returns the
// wall time of the loop in microseconds (>= 0) or -1.  On the fused hip path the choice of the
// token stays on the device and the host waits once per batch of steps (hip::GreedyDecode).
long long fr_greedy_decode(void *m, int first_id, int steps, int *out_ids) {
  long long us = -1;
  guarded([&]() {
    auto *model = static_cast<rwkv::Model *>(m);
    int id = first_id;
    const auto t0 = std::chrono::steady_clock::now();
    // the fused hip path keeps the whole loop on the device (FR_HIP_GREEDY_ON_HOST=1: token by token, as below)
    const bool chained = rwkv::hip::GreedyDecode(model, first_id, steps, out_ids);
    for (int i = 0; i < steps && !chained; i++) {
      rwkv::Tensor out = model->Run(id);
      // the fused hip path has taken the argmax on the device (first index on ties, like argmax())
      if (!rwkv::hip::device_argmax(model, out, &id))
        id = argmax(out.data_ptr<float>(), static_cast<int>(out.numel()));
      out_ids[i] = id;
    }
    const auto t1 = std::chrono::steady_clock::now();
    us = std::chrono::duration_cast<std::chrono::microseconds>(t1 - t0).count();
    return 0;
  });
  return us;
}

int fr_quantize_u8(const uint16_t *w_kn, int K, int N, uint8_t *q, uint16_t *mx, uint16_t *rx, uint16_t *my,
                   uint16_t *ry) {
  return guarded([&]() {
    rwkv::hip::quantize_u8(w_kn, K, N, q, mx, rx, my, ry);
    return 0;
  });
}

// One call of a shape / activation operator through the registry on the `hip` device, on host data:
// op 0 slice (params: start, interval, end per dimension), 1 cat (b, params[0] = dim), 2 transpose
// (params: dim_a, dim_b), 3 silu.  dtype: 0 fp32, 1 fp16, 2 int8.  Writes the result and its shape;
// returns the number of result elements.  For scripts and tests of the operator surface.
long long fr_hip_shape_op(int op, int dtype, const void *a, const int *a_shape, int a_ndim, const void *b,
                          const int *b_shape, const int *params, void *out, long long out_capacity_bytes,
                          int *out_shape, int *out_ndim) {
  return guarded([&]() -> long long {
    using namespace rwkv;
    const DType dt = dtype == 0 ? DType::kFloat32 : dtype == 1 ? DType::kFloat16 : DType::kInt8;
    auto upload = [&](const void *src, const int *shape, int nd) {
      Shape sh(shape, shape + nd);
      Tensor cpu = Tensor::Empty(sh, dt, Device::kCPU);
      std::memcpy(cpu.data_ptr(), src, cpu.nbytes());
      return Copy(cpu, Device::kHIP, true);
    };
    Tensor x = upload(a, a_shape, a_ndim), y;
    if (op == 0) {
      std::vector<Range> r;
      for (int i = 0; i < a_ndim; i++) r.emplace_back(params[3 * i], params[3 * i + 1], params[3 * i + 2]);
      y = slice(x, r);
    } else if (op == 1) {
      y = cat(x, upload(b, b_shape, a_ndim), params[0]);
    } else if (op == 2) {
      y = transpose(x, params[0], params[1]);
    } else if (op == 3) {
      y = silu(x);
    } else {
      throw FRException("unknown shape op");
    }
    Tensor h = Copy(y, Device::kCPU, true);
    if (static_cast<long long>(h.nbytes()) > out_capacity_bytes) throw FRException("result buffer too small");
    std::memcpy(out, h.data_ptr(), h.nbytes());
    *out_ndim = static_cast<int>(h.shape().size());
    for (int i = 0; i < *out_ndim; i++) out_shape[i] = static_cast<int>(h.size(i));
    return static_cast<long long>(h.numel());
  });
}

// Give the allocator's cached large blocks back to the driver; returns the bytes released.
long long fr_allocator_trim(void) {
  return guarded([&]() -> long long { return static_cast<long long>(rwkv::hip::allocator_trim()); });
}

// One raw allocation / release through the device allocator (tests of reuse, alignment and the
// out-of-memory path); fr_hip_alloc returns null and sets fr_last_error on failure.
void *fr_hip_alloc(size_t bytes) {
  void *p = nullptr;
  guarded([&]() {
    p = rwkv::allocator(rwkv::Device::kHIP).Allocate(bytes);
    return 0;
  });
  return p;
}

int fr_hip_free(void *p) {
  return guarded([&]() {
    rwkv::allocator(rwkv::Device::kHIP).Deallocate(p);
    return 0;
  });
}

int fr_allocator_stats(size_t *reserved, size_t *in_use, size_t *driver_calls) {
  return guarded([&]() {
    rwkv::hip::allocator_stats(reserved, in_use, driver_calls);
    return 0;
  });
}

}  // extern "C"
