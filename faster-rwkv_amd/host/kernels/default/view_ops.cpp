// reshape: a zero-copy view sharing storage, one dimension may be -1
// (reference: kernels/default/view_ops.cpp:10-41).  Device-independent.
#include "kernels/kernels.h"
#include "kernels/registry.h"

namespace rwkv {
namespace def {

Tensor reshape(const Tensor &x, const Shape &shape) {
  Shape out(shape);
  LengthType known = 1;
  int wildcard = -1;
  for (size_t i = 0; i < out.size(); i++) {
    if (out[i] == -1) {
      RV_CHECK(wildcard < 0) << "reshape: more than one -1";
      wildcard = static_cast<int>(i);
    } else {
      RV_CHECK(out[i] > 0) << "reshape: bad dimension " << out[i];
      known *= out[i];
    }
  }
  const LengthType total = x.numel();
  if (wildcard >= 0) {
    RV_CHECK(total % known == 0) << "reshape: " << shape_str(x.shape()) << " -> " << shape_str(shape);
    out[wildcard] = total / known;
    known *= out[wildcard];
  }
  RV_CHECK(known == total) << "reshape: " << shape_str(x.shape()) << " -> " << shape_str(shape);
  return Tensor::FromOther(x, out);
}

KernelRegister reshape_cpu("reshape", Device::kCPU, reshape);
KernelRegister reshape_hip("reshape", Device::kHIP, reshape);

}  // namespace def
}  // namespace rwkv
