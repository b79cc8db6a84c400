// rwkv::Model: strategy parsing, recurrent state, Run().  Public surface as the
// reference's model.h:14-54; "hip" is accepted as a device string.
#pragma once

#include <any>
#include <string>
#include <vector>

#include "tensor.h"

namespace rwkv {

using States = std::vector<std::vector<Tensor>>;

struct Model {
  Model(const std::string &path, const std::string &strategy);
  Model(const std::string &path, const std::string &strategy, std::any extra);
  // One id -> one-token forward; several -> seq mode.  Logits come back on the CPU (fp32).
  // On the hip device the one-token result is a view of one of two pinned host buffers: it stays
  // valid until the next-but-one Run().  Copy it to keep it longer, or set FR_HIP_OWNED_LOGITS=1
  // to get a tensor that owns its memory from every call.  A prompt (several ids) always returns
  // a tensor that owns its memory.
  Tensor Run(const std::vector<int> &ids);
  Tensor Run(int id);
  void LoadStateFile(const std::string &path);
  void SaveStateFile(const std::string &path);
  void ResetStates();
  void set_states(const States &states) { _states = states; }
  // On the hip device these are tensors over the buffers the next forward writes in place.  A copy
  // of the returned States held by the caller is a snapshot: the next forward moves the model to
  // fresh buffers first, so set_states(copy) later restores the values at the time of the copy.
  const States &states() const { return _states; }
  States &states() { return _states; }
  // Holds the number of heads, as upstream (kernels/default/init_model.cpp:67).
  int head_size() const { return _head_size; }
  int n_layer() const { return _n_layer; }
  int n_embd() const { return _n_embd; }
  int n_att() const { return _n_att; }
  int n_ffn() const { return _n_ffn; }
  const std::string &version() const { return _version; }
  const std::any &extra() const { return _extra; }
  DType weight_dtype() const { return _weight_dtype; }
  DType act_dtype() const { return _act_dtype; }
  Device act_device() const { return _act_device; }

  std::vector<Tensor> _embd_weights;  // one [n_embd] tensor per vocabulary entry

  // Backends fill these in their init_model (upstream does so through
  // `#define private public`, kernels/default/init_model.cpp:12-14).
  std::vector<Tensor> _params;  // positional, see kernels/default/init_model.cpp
  Device _act_device = Device::kCPU;
  DType _act_dtype = DType::kUndefined;
  DType _weight_dtype = DType::kUndefined;
  int _n_layer = 0, _n_embd = 0, _n_att = 0, _n_ffn = 0, _head_size = 0;
  std::string _version;
  std::any _extra;
  States _states;
};

}  // namespace rwkv
