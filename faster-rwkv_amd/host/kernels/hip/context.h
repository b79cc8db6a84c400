// State shared by the host-side files of the `hip` backend: the one stream all work is
// issued on, the table that maps a weight tensor's device pointer to the packed form
// the kernels consume, and a per-model object kept in Model::_extra.
#pragma once

#include <memory>
#include <tuple>
#include <vector>

#include "frhip.h"
#include "tensor.h"

namespace rwkv {
namespace hip {

// Initialises the device on first use and returns the backend's stream.
frhip_stream stream();

// A 2-D matmul weight as held on the device.  The Tensor that model code sees keeps the
// reference's logical shape [K, N] (tools/convert_weight.py:44-46) and a dtype of
// kFloat16 or kInt8; its data pointer is the key under which the packed description is
// found again by att / ffn / matmul.
struct PackedWeight {
  frhip_weight desc{};
  std::vector<Tensor> owners;  // device buffers: data, then mx rx my ry for uint8
  // uint8 only, made on first use by find_seq_weight: the binary16 image [N, K] of the weight
  // (frhip_dequant_u8) and its description.  Freed with the weight.
  Tensor image;
  frhip_weight image_desc{};
  bool no_image = false;  // the image could not be allocated once: not tried again
};

void register_weight(const void *data_ptr, std::shared_ptr<PackedWeight> w);
void unregister_weight(const void *data_ptr);
// nullptr when `t` is not a packed weight.
const frhip_weight *find_weight(const Tensor &t);
// The description to hand to a product over `rows` rows of activations.  The same as
// find_weight unless images are kept (FR_HIP_SEQ_IMAGE=1, or unset on a device with 128 GB
// or more; =0: never), the weight is uint8 and rows >= FRHIP_SEQ_EXPAND_ROWS: then the
// weight's binary16 image, expanded once and kept (2 more bytes per weight for as long as
// the model lives) instead of once per call into the operator's workspace.  Both ways
// multiply by the same w^, so the results are the same bits.
const frhip_weight *find_seq_weight(const Tensor &t, int rows);

// ffn_seq with the halving that follows every sixth layer folded into its last epilogue (ops.cpp); same bits as
// ffn_seq followed by scalar_div_(x, 2).
std::tuple<Tensor, Tensor> ffn_seq_div2(const Tensor &x, const Tensor &sx, const Tensor &ln_w, const Tensor &ln_b,
                                        const Tensor &k_mix, const Tensor &r_mix, const Tensor &kw, const Tensor &vw,
                                        const Tensor &rw, bool div2);

// Upload a host matrix in the reference's [K, N] layout and pack it for the kernels.
// `dtype` kFloat16: src is binary16.  kInt8: src is binary16 and is quantised on the host
// (per-column mx/rx, per-row my/ry) before upload.  Returns the tensor model code holds.
Tensor make_weight_from_host(const void *src_kn, int K, int N, DType dtype, const std::string &name);
// Same, from codes and scales already quantised (all host pointers).
Tensor make_weight_from_host_u8(const uint8_t *q_kn, const void *mx, const void *rx, const void *my,
                                const void *ry, int K, int N, const std::string &name);

// ChatRWKV-style uint8 quantisation of a [K, N] binary16 matrix on the host:
//   mx[n] = min_k w ; r = w - mx ; my[k] = min_n r ; r -= my ; rx[n] = max_k r ; r /= rx ;
//   ry[k] = max_n r ; r /= ry ; q = clamp(rint(r * 255), 0, 255)
// with mx, my, rx, ry rounded to binary16 as soon as they are formed (fp32 arithmetic,
// no contraction), so that q is exactly reproducible.
void quantize_u8(const uint16_t *w_kn, int K, int N, uint8_t *q, uint16_t *mx, uint16_t *rx, uint16_t *my,
                 uint16_t *ry);

}  // namespace hip
}  // namespace rwkv
