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
  ~ModelExtra();
};

std::shared_ptr<ModelExtra> extra_of(Model *model);

// Defined in kernels/default/model_forward.cpp
}  // namespace hip
namespace def {
Tensor ModelForward(Model *model, Device device, int id);
Tensor ModelForwardSeqFallback(Model *model, Device device, const std::vector<int> &ids, bool full_output);
}  // namespace def
}  // namespace rwkv
