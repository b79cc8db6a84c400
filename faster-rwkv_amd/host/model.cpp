#include "model.h"

#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>

#include "kernels/kernels.h"
#include "msgpack_lite.h"

namespace rwkv {

static const bool kDebug = std::getenv("FR_DEBUG") != nullptr;

static Device parse_device(const std::string &dev) {
  // reference: model.cpp:25-42, plus "hip"
  if (dev == "hip") return Device::kHIP;
  if (dev == "cpu") return Device::kCPU;
  if (dev == "cuda") return Device::kCUDA;
  if (dev == "ncnn") return Device::kNCNN;
  if (dev == "onnx") return Device::kONNX;
  if (dev == "export-ncnn") return Device::kNCNNMeta;
  if (dev == "export-onnx") return Device::kONNXMeta;
  RV_UNIMPLEMENTED() << "unknown device \"" << dev << "\"";
}

Model::Model(const std::string &path, const std::string &strategy) : Model(path, strategy, std::any()) {}

Model::Model(const std::string &path, const std::string &strategy, std::any extra) {
  const auto sp = strategy.find(' ');
  _act_device = parse_device(strategy.substr(0, sp));
  const std::string dt = sp == std::string::npos ? "" : strategy.substr(sp + 1);
  // reference: model.cpp:43-60.  ("int8"/"int4" name fp32 activations there; a backend may
  // override in init_model, and the hip backend does: its activations are fp16.)
  if (dt == "int4") {
    _act_dtype = DType::kFloat32;
    _weight_dtype = DType::kInt4;
  } else if (dt == "int8") {
    _act_dtype = DType::kFloat32;
    _weight_dtype = DType::kInt8;
  } else if (dt == "fp16") {
    _act_dtype = _weight_dtype = DType::kFloat16;
  } else if (dt == "fp32") {
    _act_dtype = _weight_dtype = DType::kFloat32;
  } else if (dt == "auto") {
    _act_dtype = _weight_dtype = DType::kUndefined;
  } else {
    RV_UNIMPLEMENTED() << "unknown dtype \"" << dt << "\"";
  }

  init_model(this, _act_device, path, strategy, extra);
  if (kDebug) {
    std::cout << "Model inited\nversion: " << _version << "\nactivation dtype: " << dtype_to_string(_act_dtype)
              << "\nweight dtype: " << dtype_to_string(_weight_dtype) << "\nhead_size: " << _head_size
              << "\nn_embd: " << _n_embd << "\nn_layer: " << _n_layer << "\nn_att: " << _n_att
              << "\nn_ffn: " << _n_ffn << std::endl;
  }
  RV_CHECK(!_version.empty());
  RV_CHECK(_act_dtype != DType::kUndefined);
  RV_CHECK(_weight_dtype != DType::kUndefined);
  RV_CHECK(_n_layer > 0);
  RV_CHECK(_n_embd > 0);
  RV_CHECK(_n_att > 0);
  if (_version.substr(0, 1) == "5") {
    RV_CHECK(_head_size > 0);
    RV_CHECK(_n_ffn > 0);
  }
  ResetStates();
}

void Model::ResetStates() {
  // reference: model.cpp:145-177.  States are built on the CPU and copied to the device.
  _states.clear();
  const Device device = (_act_device == Device::kNCNN || _act_device == Device::kONNX) ? Device::kCPU : _act_device;
  auto make = [&](const Shape &shape, DType dtype, float value) {
    Tensor t = Tensor::Empty(shape, dtype, Device::kCPU);
    return Copy(fill_(t, value), device);
  };
  for (int i = 0; i < _n_layer; i++) {
    std::vector<Tensor> s;
    if (_version == "4") {
      s.push_back(make({_n_embd}, _act_dtype, 0.f));
      s.push_back(make({_n_att}, DType::kFloat32, 0.f));
      s.push_back(make({_n_att}, DType::kFloat32, 0.f));
      s.push_back(make({_n_att}, DType::kFloat32, -1e30f));
      s.push_back(make({_n_embd}, _act_dtype, 0.f));
    } else {
      RV_CHECK(_version.substr(0, 1) == "5");
      s.push_back(make({_n_embd}, _act_dtype, 0.f));
      s.push_back(make({_head_size, _n_att / _head_size, _n_embd / _head_size}, DType::kFloat32, 0.f));
      s.push_back(make({_n_embd}, _act_dtype, 0.f));
    }
    _states.push_back(std::move(s));
  }
}

static Tensor CopyToCPUIfAvailable(const Tensor &x) {
  try {
    return Copy(x, Device::kCPU);
  } catch (std::exception &) {
    return x;
  }
}

Tensor Model::Run(const std::vector<int> &ids) {
  RV_CHECK(!ids.empty());
  if (ids.size() == 1) return CopyToCPUIfAvailable(ModelForward(this, _act_device, ids[0]));
  return CopyToCPUIfAvailable(ModelForwardSeq(this, _act_device, ids, false));
}

Tensor Model::Run(int id) { return CopyToCPUIfAvailable(ModelForward(this, _act_device, id)); }

// State files: a msgpack array (layers) of arrays (tensors) of maps {dtype, data, shape}
// (reference: model.cpp:89-143).  Device states are brought to the host first.
void Model::SaveStateFile(const std::string &path) {
  mp::Writer w;
  w.array(_states.size());
  for (const auto &layer : _states) {
    w.array(layer.size());
    for (const auto &s : layer) {
      Tensor c = Copy(s, Device::kCPU);
      w.map(3);
      w.str("dtype");
      w.str(s.dtype() == DType::kFloat32 ? "torch.float32" : s.dtype() == DType::kFloat16 ? "torch.float16" : "torch.int8");
      w.str("data");
      w.bin(c.data_ptr(), c.nbytes());
      w.str("shape");
      w.array(s.shape().size());
      for (auto d : s.shape()) w.integer(d);
    }
  }
  std::ofstream ofs(path, std::ios::binary);
  RV_CHECK(ofs.good()) << "cannot open " << path;
  ofs.write(w.buf.data(), static_cast<std::streamsize>(w.buf.size()));
}

void Model::LoadStateFile(const std::string &path) {
  std::ifstream ifs(path, std::ios::binary);
  RV_CHECK(ifs.good()) << "cannot open " << path;
  std::string data((std::istreambuf_iterator<char>(ifs)), std::istreambuf_iterator<char>());
  mp::Value root = mp::parse(data.data(), data.size());
  RV_CHECK(root.is_array() && root.arr.size() == _states.size());
  const Device device = (_act_device == Device::kNCNN || _act_device == Device::kONNX) ? Device::kCPU : _act_device;
  for (size_t i = 0; i < _states.size(); i++) {
    const mp::Value &layer = root.arr[i];
    RV_CHECK(layer.is_array() && layer.arr.size() == _states[i].size());
    for (size_t j = 0; j < _states[i].size(); j++) {
      Tensor t = mp::to_tensor(layer.arr[j]);
      RV_CHECK(t.shape() == _states[i][j].shape());
      RV_CHECK(t.dtype() == _states[i][j].dtype());
      _states[i][j] = Copy(t, device);
    }
  }
}

}  // namespace rwkv
