#include "sampler.h"

#include <algorithm>
#include <cmath>

#include "check.h"

namespace rwkv {

Sampler::Sampler() { _generator.seed(std::random_device()()); }

void Sampler::set_seed(int seed) { _generator.seed(seed); }

int Sampler::Sample(const Tensor &logits, float temperature, int top_k, float top_p) {
  RV_CHECK(logits.device() == Device::kCPU && logits.dtype() == DType::kFloat32) << "Sampler needs fp32 logits on the CPU";
  return Sample(logits.data_ptr<float>(), static_cast<int>(logits.numel()), temperature, top_k, top_p);
}

// The reference sorts all n probabilities (sampler.cpp:56-57) and then keeps a prefix.  Only
// that prefix matters, so the candidates are selected in growing blocks: the m largest are
// sorted, and m doubles until the top-p mass (or top-k) is reached inside the block.  The
// kept prefix, its order among distinct probabilities and the single generator draw are the
// same as after a full sort.
int Sampler::Sample(const float *logits, int n, float temperature, int top_k, float top_p) {
  RV_CHECK(n > 0);
  temperature = std::min(std::max(temperature, 0.1f), 5.f);  // sampler.cpp:45

  // softmax at temperature 1 (sampler.cpp:48, kernels/cpu/softmax.cpp:6-21): fp32, in index order
  _probs.resize(n);
  const float mx = *std::max_element(logits, logits + n);
  float sum = 0;
  for (int i = 0; i < n; i++) {
    _probs[i] = std::exp((logits[i] - mx) / 1.f);
    sum += _probs[i];
  }
  for (int i = 0; i < n; i++) _probs[i] /= sum;

  _cand.resize(n);
  for (int i = 0; i < n; i++) _cand[i] = {_probs[i], i};
  const auto greater = [](const std::pair<float, int> &a, const std::pair<float, int> &b) {
    return a.first > b.first || (a.first == b.first && a.second < b.second);
  };
  int len = n;
  int m = top_k > 0 ? std::min(n, top_k) : std::min(n, 64);
  for (;;) {
    std::partial_sort(_cand.begin(), _cand.begin() + m, _cand.end(), greater);
    // top-p (sampler.cpp:62-69): shortest prefix whose fp32 running sum reaches top_p
    float cumsum = 0;
    int cut = -1;
    for (int i = 0; i < m; i++) {
      cumsum += _cand[i].first;
      if (cumsum >= top_p) {
        cut = i + 1;
        break;
      }
    }
    if (cut >= 0) {
      len = cut;
      break;
    }
    if (m == n || (top_k > 0 && m >= top_k)) {  // never reached inside what top-k keeps, or at all
      len = n;
      break;
    }
    m = std::min(n, m * 4);
  }
  if (top_k > 0) len = std::min(len, top_k);  // sampler.cpp:72-74
  RV_CHECK(len <= m || m == n);

  // p^(1/T) over the kept prefix, then one draw (sampler.cpp:20-34, 88-94)
  float total = 0.f;
  for (int i = 0; i < len; i++) {
    _cand[i].first = std::pow(_cand[i].first, 1.f / temperature);
    total += _cand[i].first;
  }
  const float r = 1. * (_generator() - _generator.min()) / (_generator.max() - _generator.min()) * total;
  float cumsum = 0;
  for (int i = 0; i < len; i++) {
    cumsum += _cand[i].first;
    if (cumsum >= r) return _cand[i].second;
  }
  RV_UNIMPLEMENTED() << "Sampler: the cumulative scan ended below the draw";
  return -1;
}

}  // namespace rwkv
