// Stand-alone decode benchmark in the manner of the reference's bench_model.cpp:5-10
// (Copy(model.Run(0), kCPU) in a timing loop), without google-benchmark.
//   bench_model "<path or synthetic:...>" "hip fp16" [steps]
#include <chrono>
#include <cstdio>
#include <cstdlib>

#include "model.h"

int main(int argc, char **argv) {
  if (argc < 3) {
    std::fprintf(stderr, "usage: %s <model.fr | synthetic:spec> \"hip fp16|hip int8\" [steps]\n", argv[0]);
    return 2;
  }
  const int steps = argc > 3 ? std::atoi(argv[3]) : 128;
  try {
    rwkv::Model model(argv[1], argv[2]);
    for (int i = 0; i < 8; i++) rwkv::Copy(model.Run(0), rwkv::Device::kCPU);
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; i++) auto out = rwkv::Copy(model.Run(0), rwkv::Device::kCPU);
    const double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("%d tokens in %.3f s: %.1f tok/s, %.3f ms/token\n", steps, s, steps / s, 1e3 * s / steps);
  } catch (const std::exception &e) {
    std::fprintf(stderr, "error: %s\n", e.what());
    return 1;
  }
  return 0;
}
