// Device-generic one-token forward and the seq-mode fallback: the layer loop of the
// reference (kernels/default/model_forward.cpp:105-192, model_forward_seq.cpp:34-46)
// expressed through the operator API, so it runs on whichever device the operators are
// registered for.  The `hip` backend registers a fused, graph-replayed forward of its
// own for speed; this loop remains the plain operator-by-operator path
// (FR_HIP_GENERIC=1 selects it) and is what the two are checked against each other with.
#include "kernels/kernels.h"
#include "kernels/registry.h"
#include "model.h"

namespace rwkv {
namespace def {

Tensor ModelForward(Model *model, Device device, int id) {
  (void)device;
  auto &states = model->states();
  RV_CHECK(id >= 0 && static_cast<size_t>(id) < model->_embd_weights.size()) << "token id out of range";
  Tensor x = model->_embd_weights[id];
  const auto &p = model->_params;
  size_t pi = 0;
  const std::string &ver = model->version();
  for (size_t i = 0; i < states.size(); i++) {
    auto &st = states[i];
    if (ver == "4") {
      std::tie(x, st[0], st[1], st[2], st[3]) =
          att(x, st[0], st[1], st[2], st[3], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
              p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10]);
      pi += 11;
    } else if (ver == "5") {
      std::tie(x, st[0], st[1]) =
          att_one_v5(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                     p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12]);
      pi += 13;
    } else if (ver == "5.1" || ver == "5.2") {
      std::tie(x, st[0], st[1]) =
          att_one_v5_1(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                       p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12], p[pi + 13], p[pi + 14]);
      pi += 15;
    } else {
      RV_UNIMPLEMENTED() << "model version " << ver;
    }
    const int off = ver[0] == '5' ? 2 : 4;
    std::tie(x, st[off]) = ffn(x, st[off], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6]);
    pi += 7;
    if (x.dtype() == DType::kFloat16 && (i + 1) % 6 == 0) scalar_div_(x, 2);
  }
  x = layernorm(x, p[pi], p[pi + 1]);
  x = matmul(x, p[pi + 2]);
  if (x.dtype() == DType::kFloat16) x = cast_dtype(x, DType::kFloat32);
  return x;
}

Tensor ModelForwardSeqFallback(Model *model, Device device, const std::vector<int> &ids, bool full_output) {
  RV_CHECK(!full_output) << "full_output is not supported in fallback mode";
  RV_CHECK(!ids.empty());
  Tensor out;
  for (int id : ids) out = rwkv::ModelForward(model, device, id);
  return out;
}

KernelRegister model_forward_cpu("model_forward", Device::kCPU, ModelForward);
KernelRegister model_forward_seq_cpu("model_forward_seq", Device::kCPU, ModelForwardSeqFallback);

}  // namespace def
}  // namespace rwkv
