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

// Seq mode through the operator API, in the shape of the reference's loop
// (kernels/default/model_forward_seq.cpp:48-184): vgather of the embedding rows, per layer the seq
// attention operator of the model's version and ffn_seq, the /2 rescale of fp16 activations every
// sixth layer, then the last row (slice + squeeze, :170-172) through ln_out, head and the cast.
// RWKV-4 goes through `att_seq`, which upstream lacks (:111-112 throws); RWKV-5.1 has no seq
// operator upstream either (:127-128) and runs as one-token steps.
Tensor ModelForwardSeq(Model *model, Device device, const std::vector<int> &ids, bool full_output) {
  const std::string &ver = model->version();
  if (ver == "5.1") return ModelForwardSeqFallback(model, device, ids, full_output);
  RV_CHECK(!ids.empty());
  auto &states = model->states();
  const auto &p = model->_params;
  Tensor x = vgather(model->_embd_weights, ids);
  size_t pi = 0;
  for (size_t i = 0; i < states.size(); i++) {
    auto &st = states[i];
    if (ver == "4") {
      std::tie(x, st[0], st[1], st[2], st[3]) =
          att_seq(x, st[0], st[1], st[2], st[3], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5],
                  p[pi + 6], p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10]);
      pi += 11;
    } else if (ver == "5") {
      std::tie(x, st[0], st[1]) =
          att_seq_v5(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                     p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12]);
      pi += 13;
    } else if (ver == "5.2") {
      std::tie(x, st[0], st[1]) =
          att_seq_v5_2(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                       p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12], p[pi + 13], p[pi + 14],
                       model->n_att());
      pi += 15;
    } else {
      RV_UNIMPLEMENTED() << "model version " << ver;
    }
    const int off = ver[0] == '5' ? 2 : 4;
    std::tie(x, st[off]) = ffn_seq(x, st[off], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6]);
    pi += 7;
    if (x.dtype() == DType::kFloat16 && (i + 1) % 6 == 0) scalar_div_(x, 2);
  }
  if (!full_output) x = x.slice({Range(-1, 1, static_cast<int>(x.size(0))), Range::All}).squeeze(0);
  x = layernorm(x, p[pi], p[pi + 1]);
  x = matmul(x, p[pi + 2]);
  if (x.dtype() == DType::kFloat16) x = cast_dtype(x, DType::kFloat32);
  return x;
}

KernelRegister model_forward_cpu("model_forward", Device::kCPU, ModelForward);
KernelRegister model_forward_seq_cpu("model_forward_seq", Device::kCPU, ModelForwardSeqFallback);

}  // namespace def
}  // namespace rwkv
