// The operator API: thin inline dispatchers that look the implementation up in the
// registry under (name, device of the first tensor argument).
//
// Names, argument order and return types are those of the reference's
// kernels/kernels.h (att :15-24, att_one_v5 :26-37, att_seq_v5 :39-50, att_one_v5_1
// :52-63, att_seq_v5_2 :65-76, ffn :80-87, ffn_seq :89-96, primitives :98-266,
// init_model / ModelForward / ModelForwardSeq / allocator :268-289), so a backend
// registered here is found by unchanged model code.  `att_seq` (RWKV-4 sequence
// attention) is an addition: the reference has no such operator
// (kernels/default/model_forward_seq.cpp:111-112).
#pragma once

#include <any>
#include <string>
#include <tuple>
#include <vector>

#include "check.h"
#include "kernels/allocator.h"
#include "kernels/registry.h"
#include "tensor.h"

namespace rwkv {

using T1 = Tensor;
using T2 = std::tuple<Tensor, Tensor>;
using T3 = std::tuple<Tensor, Tensor, Tensor>;
using T5 = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor>;
using CT = const Tensor &;

// FR_OP(ret, name, "registry key", device expression, (params), (call args))
#define FR_OP(RET, NAME, KEY, DEV, PARAMS, ARGS)                                   \
  inline RET NAME PARAMS {                                                         \
    return KernelRegistry::Instance().Get<RET(*) PARAMS>(KEY, DEV) ARGS;           \
  }

// ---- fused layer operators ---------------------------------------------------
FR_OP(T5, att, "att", x.device(),
      (CT x, CT sx, CT aa, CT bb, CT pp, CT ln_w, CT ln_b, CT k_mix, CT v_mix, CT r_mix, CT t_decay, CT t_first,
       CT kw, CT vw, CT rw, CT ow),
      (x, sx, aa, bb, pp, ln_w, ln_b, k_mix, v_mix, r_mix, t_decay, t_first, kw, vw, rw, ow))

FR_OP(T5, att_seq, "att_seq", x.device(),
      (CT x, CT sx, CT aa, CT bb, CT pp, CT ln_w, CT ln_b, CT k_mix, CT v_mix, CT r_mix, CT t_decay, CT t_first,
       CT kw, CT vw, CT rw, CT ow),
      (x, sx, aa, bb, pp, ln_w, ln_b, k_mix, v_mix, r_mix, t_decay, t_first, kw, vw, rw, ow))

#define FR_V5_PARAMS                                                                                             \
  (CT x, CT sx, CT s, CT ln_w, CT ln_b, CT lx_w, CT lx_b, CT k_mix, CT v_mix, CT r_mix, CT t_decay, CT t_first, \
   CT kw, CT vw, CT rw, CT ow)
#define FR_V5_ARGS (x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, t_decay, t_first, kw, vw, rw, ow)
FR_OP(T3, att_one_v5, "att_one_v5", x.device(), FR_V5_PARAMS, FR_V5_ARGS)
FR_OP(T3, att_seq_v5, "att_seq_v5", x.device(), FR_V5_PARAMS, FR_V5_ARGS)

#define FR_V51_PARAMS                                                                                  \
  (CT x, CT sx, CT s, CT ln_w, CT ln_b, CT lx_w, CT lx_b, CT k_mix, CT v_mix, CT r_mix, CT g_mix,     \
   CT t_decay, CT t_first, CT kw, CT vw, CT rw, CT gw, CT ow)
#define FR_V51_ARGS \
  (x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay, t_first, kw, vw, rw, gw, ow)
FR_OP(T3, att_one_v5_1, "att_one_v5_1", x.device(), FR_V51_PARAMS, FR_V51_ARGS)

FR_OP(T3, att_seq_v5_2, "att_seq_v5_2", x.device(),
      (CT x, CT sx, CT s, CT ln_w, CT ln_b, CT lx_w, CT lx_b, CT k_mix, CT v_mix, CT r_mix, CT g_mix, CT t_decay,
       CT t_first, CT kw, CT vw, CT rw, CT gw, CT ow, int n_att),
      (x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay, t_first, kw, vw, rw, gw, ow, n_att))

#define FR_FFN_PARAMS (CT x, CT sx, CT ln_w, CT ln_b, CT k_mix, CT r_mix, CT kw, CT vw, CT rw)
#define FR_FFN_ARGS (x, sx, ln_w, ln_b, k_mix, r_mix, kw, vw, rw)
FR_OP(T2, ffn, "ffn", x.device(), FR_FFN_PARAMS, FR_FFN_ARGS)
FR_OP(T2, ffn_seq, "ffn_seq", x.device(), FR_FFN_PARAMS, FR_FFN_ARGS)

// ---- primitives ----------------------------------------------------------------
FR_OP(T1, cast_dtype, "cast_dtype", x.device(), (CT x, DType dtype), (x, dtype))
FR_OP(Tensor &, fill_, "fill_", x.device(), (Tensor & x, float val), (x, val))
FR_OP(T1, scalar_div_, "scalar_div_", x.device(), (Tensor & x, float val), (x, val))
FR_OP(T1, layernorm, "layernorm", x.device(), (CT x, CT weight, CT bias), (x, weight, bias))
FR_OP(T1, groupnorm, "groupnorm", x.device(), (CT x, int num_groups, CT weight, CT bias),
      (x, num_groups, weight, bias))
FR_OP(T1, matmul, "matmul", a.device(), (CT a, CT b), (a, b))
FR_OP(T1, cat, "cat", a.device(), (CT a, CT b, int dim), (a, b, dim))
FR_OP(T1, add, "add", default_dispatch_device().value_or(x.device()), (CT x, CT y), (x, y))
FR_OP(T1, sub, "rsub_scalar", default_dispatch_device().value_or(y.device()), (float x, CT y), (x, y))
FR_OP(T1, sub, "sub", x.device(), (CT x, CT y), (x, y))
FR_OP(T1, mul, "mul", default_dispatch_device().value_or(x.device()), (CT x, CT y), (x, y))
FR_OP(T1, div, "div", x.device(), (CT x, CT y), (x, y))
FR_OP(T1, exp, "exp", x.device(), (CT x), (x))
FR_OP(T1, relu, "relu", x.device(), (CT x), (x))
FR_OP(T1, sigmoid, "sigmoid", x.device(), (CT x), (x))
FR_OP(T1, silu, "silu", x.device(), (CT x), (x))
FR_OP(T1, maximum, "maximum", x.device(), (CT x, CT y), (x, y))
FR_OP(T1, softmax, "softmax", x.device(), (CT x, float temperature), (x, temperature))
FR_OP(T1, reshape, "reshape", x.device(), (CT x, const Shape &shape), (x, shape))
FR_OP(T1, slice, "slice", x.device(), (CT x, const std::vector<Range> &ranges), (x, ranges))
FR_OP(T1, transpose, "transpose", x.device(), (CT x, int dim_a, int dim_b), (x, dim_a, dim_b))

// All tensors of `x` must have the same shape (rows of the embedding table).
inline Tensor vgather(const std::vector<Tensor> &x, const std::vector<int> &idx) {
  RV_CHECK(!x.empty());
  using Fn = Tensor (*)(const std::vector<Tensor> &, const std::vector<int> &);
  return KernelRegistry::Instance().Get<Fn>("vgather", x[0].device())(x, idx);
}

inline Tensor flatten(CT x) { return reshape(x, {x.numel()}); }

inline Tensor unsqueeze(CT x, int dim) {
  Shape s = x.shape();
  if (dim < 0) dim += static_cast<int>(s.size());  // as upstream (kernels.h:188-190)
  RV_CHECK(dim >= 0 && dim <= static_cast<int>(s.size()));
  s.insert(s.begin() + dim, 1);
  return reshape(x, s);
}

inline Tensor squeeze(CT x, int dim) {
  Shape s = x.shape();
  if (dim < 0) dim += static_cast<int>(s.size());
  RV_CHECK(dim >= 0 && dim < static_cast<int>(s.size()));
  s.erase(s.begin() + dim);
  return reshape(x, s);
}

// ---- model-level entry points ----------------------------------------------------
class Model;

inline void init_model(Model *model, Device device, const std::string &path, const std::string &strategy,
                       const std::any &extra) {
  using Fn = void (*)(Model *, Device, const std::string &, const std::string &, const std::any &);
  KernelRegistry::Instance().Get<Fn>("init_model", device)(model, device, path, strategy, extra);
}

inline Tensor ModelForward(Model *model, Device device, int id) {
  using Fn = Tensor (*)(Model *, Device, int);
  return KernelRegistry::Instance().Get<Fn>("model_forward", device)(model, device, id);
}

inline Tensor ModelForwardSeq(Model *model, Device device, const std::vector<int> &id, bool full_output) {
  using Fn = Tensor (*)(Model *, Device, const std::vector<int> &, bool);
  return KernelRegistry::Instance().Get<Fn>("model_forward_seq", device)(model, device, id, full_output);
}

inline Allocator &allocator(Device device) {
  return KernelRegistry::Instance().Get<Allocator &(*)()>("allocator", device)();
}

#undef FR_OP

}  // namespace rwkv
