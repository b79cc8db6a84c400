// Token sampler with the interface and the arithmetic of the reference's Sampler
// (sampler.h:8-16, sampler.cpp:18-101): softmax at temperature 1, descending sort, top-p cut,
// top-k cut, p^(1/temperature) re-weighting, one draw from std::minstd_rand0 through a
// hand-made cumulative scan so that a seed gives the same tokens on every platform.
#pragma once

#include <random>
#include <utility>
#include <vector>

#include "tensor.h"

namespace rwkv {

class Sampler {
 public:
  Sampler();
  // logits: fp32 tensor on the CPU (what Model::Run returns).
  int Sample(const Tensor &logits, float temperature, int top_k, float top_p);
  // Same on a raw buffer.
  int Sample(const float *logits, int n, float temperature, int top_k, float top_p);
  void set_seed(int seed);

 private:
  std::minstd_rand0 _generator;
  std::vector<float> _probs;
  std::vector<std::pair<float, int>> _cand;
};

}  // namespace rwkv
