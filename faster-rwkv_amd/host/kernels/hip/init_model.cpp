// init_model for Device::kHIP: builds Model::_params (positional, as
// kernels/default/init_model.cpp:75-126) and the embedding rows on the device, from
//   * a `.fr` file (msgpack written by tools/convert_weight.py:12-55), or
//   * a synthetic specification "synthetic:v=4,L=24,C=2048,F=8192,V=65536,seed=1"
//     (random-init weights of a given architecture; benchmarks and tests).
// Matrix weights are packed output-major; with the "int8" strategy binary16 matrices are
// quantised to uint8 with per-column/per-row offsets and ranges on the way in, and
// pre-quantised files (`<name>` uint8 plus `<name>_mx/_rx/_my/_ry`) are taken as they are.
// Activations are fp16 on this backend whatever the strategy's dtype word says.
#include <cmath>
#include <functional>
#include <cstdlib>
#include <fstream>
#include <map>
#include <thread>

#include "kernels/hip/context.h"
#include "kernels/hip/hip_model.h"
#include "kernels/kernels.h"
#include "kernels/registry.h"
#include "model.h"
#include "msgpack_lite.h"

namespace rwkv {
namespace hip {

ModelExtra::~ModelExtra() {
  for (const void *p : packed) unregister_weight(p);
}

std::shared_ptr<ModelExtra> extra_of(Model *model) {
  auto *sp = std::any_cast<std::shared_ptr<ModelExtra>>(&model->_extra);
  RV_CHECK(sp != nullptr) << "model was not initialised by the hip backend";
  return *sp;
}

namespace {

// ---- deterministic generator: splitmix64 counters -> uniform / Box-Muller normal ----
inline uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}
inline float u01(uint64_t key, uint64_t i) {  // (0, 1]
  return (static_cast<float>(splitmix64(key + i) >> 40) + 1.0f) * (1.0f / 16777216.0f);
}
inline float normal(uint64_t key, uint64_t i) {
  const float u1 = u01(key, 2 * i), u2 = u01(key, 2 * i + 1);
  return std::sqrt(-2.0f * std::log(u1)) * std::cos(6.28318530717958647692f * u2);
}

void parallel_rows(int64_t n, const std::function<void(int64_t, int64_t)> &fn) {
  int nt = static_cast<int>(std::thread::hardware_concurrency());
  nt = std::max(1, std::min(nt, 16));
  if (n < 1024) nt = 1;
  std::vector<std::thread> th;
  for (int t = 0; t < nt; t++) th.emplace_back([=, &fn]() { fn(n * t / nt, n * (t + 1) / nt); });
  for (auto &t : th) t.join();
}

struct Spec {
  std::string version = "4";
  int L = 0, C = 0, F = 0, V = 0, H = 0;
  uint64_t seed = 0;
};

Spec parse_spec(const std::string &s) {
  Spec sp;
  size_t pos = 0;
  while (pos < s.size()) {
    size_t comma = s.find(',', pos);
    if (comma == std::string::npos) comma = s.size();
    const std::string kv = s.substr(pos, comma - pos);
    const size_t eq = kv.find('=');
    RV_CHECK(eq != std::string::npos) << "synthetic spec: expected key=value, got " << kv;
    const std::string k = kv.substr(0, eq), v = kv.substr(eq + 1);
    if (k == "v") sp.version = v;
    else if (k == "L") sp.L = std::atoi(v.c_str());
    else if (k == "C") sp.C = std::atoi(v.c_str());
    else if (k == "F") sp.F = std::atoi(v.c_str());
    else if (k == "V") sp.V = std::atoi(v.c_str());
    else if (k == "H") sp.H = std::atoi(v.c_str());
    else if (k == "seed") sp.seed = std::strtoull(v.c_str(), nullptr, 10);
    else RV_UNIMPLEMENTED() << "synthetic spec: unknown key " << k;
    pos = comma + 1;
  }
  RV_CHECK(sp.L > 0 && sp.C > 0 && sp.F > 0 && sp.V > 0) << "synthetic spec needs L, C, F, V";
  if (sp.version[0] == '5') RV_CHECK(sp.H > 0 && sp.C % sp.H == 0) << "synthetic spec: v5 needs H dividing C";
  return sp;
}

Tensor vec_to_device(const std::vector<float> &v, const Shape &shape, DType dtype, const std::string &name) {
  Tensor c = Tensor::Empty(shape, dtype, Device::kCPU);
  if (dtype == DType::kFloat16) {
    float16 *p = c.data_ptr<float16>();
    for (size_t i = 0; i < v.size(); i++) p[i] = float16(v[i]);
  } else {
    std::memcpy(c.data_ptr(), v.data(), v.size() * 4);
  }
  Tensor d = Copy(c, Device::kHIP, true);
  d.name = name;
  d.is_constant = true;
  return d;
}

// Random-init model: 2-D weights ~N(0, 0.02); time_decay_raw ~U(-5,1) (v4) or U(-6,0)
// (v5.2); time_first ~U(-1,1); time_mix ~U(0,1); layernorm gamma 1, beta 0.  Stored forms
// are the ones the kernels consume: v4 time_decay = -exp(raw); v5.2 time_decay =
// exp(-exp(raw)) of shape [H, S].  Embedding rows ~N(0, 0.02) passed through a layernorm
// (the converter folds ln0 into the table).
void build_synthetic(Model *model, const Spec &sp, DType wdtype, ModelExtra &ex) {
  const int C = sp.C, F = sp.F, V = sp.V, L = sp.L;
  const bool v5 = sp.version[0] == '5';
  const bool v50 = sp.version == "5";  // RWKV-5.0: no gate, one decay / bonus per head
  uint64_t stream_id = 0;
  auto key = [&]() { return splitmix64(sp.seed * 0x100000001B3ull + (++stream_id)); };
  auto push = [&](Tensor t) { model->_params.push_back(std::move(t)); };
  auto matrix = [&](int K, int N, const std::string &name) {
    const uint64_t k = key();
    std::vector<uint16_t> w(static_cast<size_t>(K) * N);
    parallel_rows(static_cast<int64_t>(w.size()), [&](int64_t lo, int64_t hi) {
      for (int64_t i = lo; i < hi; i++) w[i] = float16(0.02f * normal(k, static_cast<uint64_t>(i))).bits;
    });
    Tensor t = make_weight_from_host(w.data(), K, N, wdtype, name);
    ex.packed.push_back(t.data_ptr());
    push(t);
  };
  auto constant = [&](int n, float v, DType dt, const std::string &name) {
    push(vec_to_device(std::vector<float>(n, v), {n}, dt, name));
  };
  auto uniform = [&](int n, float lo, float hi, DType dt, const Shape &shape, const std::string &name,
                     int transform = 0) {
    const uint64_t k = key();
    std::vector<float> v(n);
    for (int i = 0; i < n; i++) {
      float u = lo + (hi - lo) * u01(k, i);
      if (transform == 1) u = -std::exp(u);
      if (transform == 2) u = std::exp(-std::exp(u));
      v[i] = u;
    }
    push(vec_to_device(v, shape, dt, name));
  };
  const DType act = DType::kFloat16;
  for (int l = 0; l < L; l++) {
    const std::string b = "blocks." + std::to_string(l) + ".";
    constant(C, 1.f, act, b + "ln1.weight");
    constant(C, 0.f, act, b + "ln1.bias");
    if (v5) {
      constant(C, 1.f, DType::kFloat32, b + "att.ln_x.weight");
      constant(C, 0.f, DType::kFloat32, b + "att.ln_x.bias");
    }
    uniform(C, 0, 1, act, {C}, b + "att.time_mix_k");
    uniform(C, 0, 1, act, {C}, b + "att.time_mix_v");
    uniform(C, 0, 1, act, {C}, b + "att.time_mix_r");
    if (v5 && !v50) uniform(C, 0, 1, act, {C}, b + "att.time_mix_g");
    if (v50) {
      uniform(sp.H, -6, 0, DType::kFloat32, {sp.H}, b + "att.time_decay", 2);
      uniform(sp.H, -1, 1, DType::kFloat32, {sp.H}, b + "att.time_first");
    } else if (v5) {
      uniform(C, -6, 0, DType::kFloat32, {sp.H, C / sp.H}, b + "att.time_decay", 2);
      uniform(C, -1, 1, DType::kFloat32, {sp.H, C / sp.H}, b + "att.time_first");
    } else {
      uniform(C, -5, 1, DType::kFloat32, {C}, b + "att.time_decay", 1);
      uniform(C, -1, 1, DType::kFloat32, {C}, b + "att.time_first");
    }
    matrix(C, C, b + "att.key.weight");
    matrix(C, C, b + "att.value.weight");
    matrix(C, C, b + "att.receptance.weight");
    if (v5 && !v50) matrix(C, C, b + "att.gate.weight");
    matrix(C, C, b + "att.output.weight");
    constant(C, 1.f, act, b + "ln2.weight");
    constant(C, 0.f, act, b + "ln2.bias");
    uniform(C, 0, 1, act, {C}, b + "ffn.time_mix_k");
    uniform(C, 0, 1, act, {C}, b + "ffn.time_mix_r");
    matrix(C, F, b + "ffn.key.weight");
    matrix(F, C, b + "ffn.value.weight");
    matrix(C, C, b + "ffn.receptance.weight");
  }
  constant(C, 1.f, act, "ln_out.weight");
  constant(C, 0.f, act, "ln_out.bias");
  matrix(C, V, "head.weight");

  // embedding table: one slab, rows normalised to zero mean / unit variance
  const uint64_t k = key();
  Tensor emb_cpu = Tensor::Empty({V, C}, act, Device::kCPU);
  float16 *e = emb_cpu.data_ptr<float16>();
  parallel_rows(V, [&](int64_t lo, int64_t hi) {
    std::vector<float> row(C);
    for (int64_t r = lo; r < hi; r++) {
      double s = 0, q = 0;
      for (int c = 0; c < C; c++) {
        row[c] = 0.02f * normal(k, static_cast<uint64_t>(r) * C + c);
        s += row[c];
      }
      const double mean = s / C;
      for (int c = 0; c < C; c++) q += (row[c] - mean) * (row[c] - mean);
      const double inv = 1.0 / std::sqrt(q / C + 1e-5);
      for (int c = 0; c < C; c++) e[r * C + c] = float16(static_cast<float>((row[c] - mean) * inv));
    }
  });
  ex.emb_table = Copy(emb_cpu, Device::kHIP, true);
  model->_n_layer = L;
  model->_n_embd = C;
  model->_n_att = C;
  model->_n_ffn = F;
  model->_head_size = sp.H;
  model->_version = sp.version;
}

bool is_matrix_name(const std::string &n) {
  auto ends = [&](const char *suf) {
    const std::string s(suf);
    return n.size() >= s.size() && n.compare(n.size() - s.size(), s.size(), s) == 0;
  };
  return ends("key.weight") || ends("value.weight") || ends("receptance.weight") || ends("output.weight") ||
         ends("gate.weight") || n == "head.weight";
}

void build_from_fr(Model *model, const std::string &path, DType wdtype, ModelExtra &ex) {
  std::ifstream ifs(path, std::ios::binary);
  RV_CHECK(ifs.good()) << "cannot open model file " << path;
  std::string data((std::istreambuf_iterator<char>(ifs)), std::istreambuf_iterator<char>());
  mp::Value root = mp::parse(data.data(), data.size());
  RV_CHECK(root.is_map()) << ".fr file: top level is not a map";
  const mp::Value &weights = root.at("weights");
  RV_CHECK(weights.is_map());
  std::map<std::string, const mp::Value *> by_name;
  for (const auto &kv : weights.map) by_name[kv.first.as_str()] = &kv.second;

  model->_n_layer = static_cast<int>(root.at("n_layer").as_int());
  model->_n_embd = static_cast<int>(root.at("n_embd").as_int());
  model->_version = root.find("version") ? root.at("version").as_str() : "4";
  if (model->_version[0] == '5') {
    model->_head_size = static_cast<int>(root.at("n_head").as_int());
    model->_n_att = static_cast<int>(root.at("n_att").as_int());
    model->_n_ffn = static_cast<int>(root.at("n_ffn").as_int());
  } else {
    RV_CHECK(model->_version == "4");
    model->_n_att = model->_n_embd;
  }

  auto push_param = [&](const std::string &key) {
    auto it = by_name.find(key);
    RV_CHECK(it != by_name.end()) << ".fr file: missing tensor " << key;
    Tensor cpu = mp::to_tensor(*it->second);
    if (is_matrix_name(key)) {
      RV_CHECK(cpu.shape().size() == 2);
      const int K = static_cast<int>(cpu.size(0)), N = static_cast<int>(cpu.size(1));
      Tensor t;
      if (cpu.dtype() == DType::kInt8) {  // pre-quantised: codes + <key>_mx/_rx/_my/_ry
        Tensor sc[4];
        const char *suf[4] = {"_mx", "_rx", "_my", "_ry"};
        for (int i = 0; i < 4; i++) {
          auto s = by_name.find(key + suf[i]);
          RV_CHECK(s != by_name.end()) << ".fr file: uint8 tensor " << key << " without " << suf[i];
          sc[i] = mp::to_tensor(*s->second);
          RV_CHECK(sc[i].dtype() == DType::kFloat16 && sc[i].numel() == ((i < 2) ? N : K));
        }
        t = make_weight_from_host_u8(static_cast<const uint8_t *>(cpu.data_ptr()), sc[0].data_ptr(),
                                     sc[1].data_ptr(), sc[2].data_ptr(), sc[3].data_ptr(), K, N, key);
      } else {
        if (cpu.dtype() == DType::kFloat32) cpu = cast_dtype(cpu, DType::kFloat16);
        t = make_weight_from_host(cpu.data_ptr(), K, N, wdtype, key);
      }
      if (key == "ffn.key.weight" || key.find(".ffn.key.weight") != std::string::npos) model->_n_ffn = N;
      ex.packed.push_back(t.data_ptr());
      model->_params.push_back(t);
    } else {
      // vectors: time_decay / time_first / ln_x stay fp32 (the WKV and groupnorm kernels read
      // fp32); everything else is brought to the activation dtype
      const bool keep_f32 = key.find("time_decay") != std::string::npos ||
                            key.find("time_first") != std::string::npos || key.find("ln_x") != std::string::npos;
      const DType want = keep_f32 ? DType::kFloat32 : DType::kFloat16;
      if (cpu.dtype() != want) cpu = cast_dtype(cpu, want);
      Tensor t = Copy(cpu, Device::kHIP, true);
      t.name = key;
      t.is_constant = true;
      model->_params.push_back(t);
    }
  };
  const std::string &ver = model->_version;
  for (int i = 0; i < model->_n_layer; i++) {
    const std::string b = "blocks." + std::to_string(i) + ".", a = b + "att.", f = b + "ffn.";
    push_param(b + "ln1.weight");
    push_param(b + "ln1.bias");
    if (ver[0] == '5') {
      push_param(a + "ln_x.weight");
      push_param(a + "ln_x.bias");
    }
    push_param(a + "time_mix_k");
    push_param(a + "time_mix_v");
    push_param(a + "time_mix_r");
    if (ver == "5.1" || ver == "5.2") push_param(a + "time_mix_g");
    push_param(a + "time_decay");
    push_param(a + "time_first");
    push_param(a + "key.weight");
    push_param(a + "value.weight");
    push_param(a + "receptance.weight");
    if (ver == "5.1" || ver == "5.2") push_param(a + "gate.weight");
    push_param(a + "output.weight");
    push_param(b + "ln2.weight");
    push_param(b + "ln2.bias");
    push_param(f + "time_mix_k");
    push_param(f + "time_mix_r");
    push_param(f + "key.weight");
    push_param(f + "value.weight");
    push_param(f + "receptance.weight");
  }
  push_param("ln_out.weight");
  push_param("ln_out.bias");
  push_param("head.weight");

  const mp::Value &embd = root.at("embd_weights");
  RV_CHECK(embd.is_array() && !embd.arr.empty());
  const int V = static_cast<int>(embd.arr.size()), C = model->_n_embd;
  Tensor emb_cpu = Tensor::Empty({V, C}, DType::kFloat16, Device::kCPU);
  for (int r = 0; r < V; r++) {
    Tensor row = mp::to_tensor(embd.arr[r]);
    RV_CHECK(row.numel() == C);
    if (row.dtype() != DType::kFloat16) row = cast_dtype(row, DType::kFloat16);
    std::memcpy(emb_cpu.data_ptr<float16>() + static_cast<size_t>(r) * C, row.data_ptr(), 2 * static_cast<size_t>(C));
  }
  ex.emb_table = Copy(emb_cpu, Device::kHIP, true);
}

}  // namespace

void init_model(Model *model, Device device, const std::string &path, const std::string &strategy,
                const std::any & /*extra*/) {
  RV_CHECK(device == Device::kHIP);
  stream();
  const std::string dt = strategy.substr(strategy.find(' ') + 1);
  RV_CHECK(dt == "fp16" || dt == "int8") << "hip backend: strategy must be \"hip fp16\" or \"hip int8\", got \""
                                         << strategy << "\"";
  const DType wdtype = dt == "int8" ? DType::kInt8 : DType::kFloat16;
  auto ex = std::make_shared<ModelExtra>();
  const std::string tag = "synthetic:";
  if (path.compare(0, tag.size(), tag) == 0)
    build_synthetic(model, parse_spec(path.substr(tag.size())), wdtype, *ex);
  else
    build_from_fr(model, path, wdtype, *ex);
  model->_act_dtype = DType::kFloat16;  // model.cpp:46-49 names fp32 for "int8"; this backend computes in fp16
  model->_weight_dtype = wdtype;
  // embedding rows: views into the slab (the reference allocates one tensor per row,
  // kernels/default/init_model.cpp:128-132)
  const int V = static_cast<int>(ex->emb_table.size(0)), C = model->_n_embd;
  char *base = static_cast<char *>(ex->emb_table.data_ptr());
  model->_embd_weights.reserve(V);
  for (int r = 0; r < V; r++)
    model->_embd_weights.push_back(Tensor::FromPtr(base + static_cast<size_t>(r) * C * 2, {C}, DType::kFloat16, Device::kHIP));
  model->_extra = ex;
}

KernelRegister init_model_reg("init_model", Device::kHIP, init_model);

}  // namespace hip
}  // namespace rwkv
