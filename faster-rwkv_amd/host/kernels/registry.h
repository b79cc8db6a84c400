// Operator registry: (name, device) -> type-erased function pointer, filled by static
// KernelRegister objects (reference: kernels/registry.h:11-35).  Get<T> must be asked
// for exactly the pointer type that was registered; asking for another throws
// std::bad_any_cast, an unknown key throws std::runtime_error("kernel <name> not found").
#pragma once

#include <any>
#include <map>
#include <stdexcept>
#include <string>
#include <utility>

#include "tensor.h"

namespace rwkv {

class KernelRegistry {
public:
  static KernelRegistry &Instance();
  // Last registration for a key wins; `priority` is accepted and ignored, as upstream.
  void Register(const std::string &name, Device device, std::any kernel, int priority);
  bool Has(const std::string &name, Device device) const;
  template <typename T> T Get(const std::string &name, Device device) const {
    auto it = _table.find({name, device});
    if (it == _table.end()) throw std::runtime_error("kernel " + name + " not found");
    return std::any_cast<T>(it->second);
  }

private:
  std::map<std::pair<std::string, Device>, std::any> _table;
};

struct KernelRegister {
  KernelRegister(const std::string &name, Device device, std::any kernel, int priority = 1) {
    KernelRegistry::Instance().Register(name, device, std::move(kernel), priority);
  }
};

}  // namespace rwkv
