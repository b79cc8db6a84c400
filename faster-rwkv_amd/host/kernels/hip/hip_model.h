// Per-model state of the `hip` backend, kept in Model::_extra.
#pragma once

#include <memory>
#include <vector>

#include "frhip.h"
#include "tensor.h"

namespace rwkv {
class Model;
namespace hip {

struct DecodePlan;  // fused one-token forward: buffers + captured graphs (model_forward.cpp)

struct ModelExtra {
  Tensor emb_table;                 // [V, C]: one slab; Model::_embd_weights are row views into it
  std::vector<const void *> packed; // keys registered in the weight table, released with the model
  std::shared_ptr<DecodePlan> plan;
  int32_t last_argmax = -1;               // index of the largest logit of the last fused one-token pass ...
  const void *last_argmax_of = nullptr;   // ... and the logits buffer it belongs to
  ~ModelExtra();
};

std::shared_ptr<ModelExtra> extra_of(Model *model);
bool device_argmax(Model *model, const Tensor &logits, int *id);
// `steps` greedy tokens from `first_id` with the token choice left on the device (model_forward.cpp).
bool GreedyDecode(Model *model, int first_id, int steps, int *out_ids, Tensor *last_logits = nullptr);

// Defined in kernels/default/model_forward.cpp
}  // namespace hip
namespace def {
Tensor ModelForward(Model *model, Device device, int id);
Tensor ModelForwardSeq(Model *model, Device device, const std::vector<int> &ids, bool full_output);
Tensor ModelForwardSeqFallback(Model *model, Device device, const std::vector<int> &ids, bool full_output);
}  // namespace def
}  // namespace rwkv
