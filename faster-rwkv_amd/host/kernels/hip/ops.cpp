// Operators registered for Device::kHIP.  Each is a thin host function: it checks
// shapes, allocates outputs through the device allocator, and calls the C ABI of
// libfrhip.so with raw pointers.  Signatures are the ones kernels/kernels.h dispatches to.
#include <cstring>

#include "kernels/hip/context.h"
#include "kernels/kernels.h"
#include "kernels/registry.h"

namespace rwkv {
namespace hip {

namespace {

int to_frhip_dtype(DType d) {
  if (d == DType::kFloat16) return FRHIP_F16;
  if (d == DType::kFloat32) return FRHIP_F32;
  if (d == DType::kInt8) return FRHIP_U8;
  RV_UNIMPLEMENTED() << "dtype " << dtype_to_string(d) << " on hip";
}

// Packed description of a weight tensor.  A tensor that did not come from init_model
// (a plain [K, N] binary16 matrix on the device) is packed on the fly into `tmp`.
// `rows`: rows of activations the product will have (1 for the one-token operators).
const frhip_weight *weight_of(const Tensor &w, frhip_weight &tmp_desc, Tensor &tmp, int rows = 1) {
  if (const frhip_weight *p = find_seq_weight(w, rows)) return p;
  RV_CHECK(w.shape().size() == 2 && w.dtype() == DType::kFloat16)
      << "matmul on hip: right operand must be a packed weight or a 2-D fp16 tensor";
  const int K = static_cast<int>(w.size(0)), N = static_cast<int>(w.size(1));
  tmp = Tensor::Empty({N, K}, DType::kFloat16, Device::kHIP);
  FRHIP_CHECK(frhip_pack_transpose(w.data_ptr(), tmp.data_ptr(), K, N, 2, stream()));
  std::memset(&tmp_desc, 0, sizeof(tmp_desc));
  tmp_desc.data = tmp.data_ptr();
  tmp_desc.K = K;
  tmp_desc.N = N;
  tmp_desc.dtype = FRHIP_F16;
  return &tmp_desc;
}

Tensor workspace(int C, int F) {
  const size_t bytes = frhip_decode_workspace_bytes(C, F);
  return Tensor::Empty({static_cast<LengthType>(bytes)}, DType::kInt8, Device::kHIP);
}

}  // namespace

Tensor &fill_(Tensor &x, float value) {
  FRHIP_CHECK(frhip_fill(x.data_ptr(), to_frhip_dtype(x.dtype()), value, static_cast<size_t>(x.numel()), stream()));
  return x;
}

Tensor cast_dtype(const Tensor &x, DType dtype) {
  if (x.dtype() == dtype) return x;
  Tensor y = Tensor::Empty(x.shape(), dtype, Device::kHIP);
  FRHIP_CHECK(frhip_cast(x.data_ptr(), to_frhip_dtype(x.dtype()), y.data_ptr(), to_frhip_dtype(dtype),
                         static_cast<size_t>(x.numel()), stream()));
  return y;
}

Tensor scalar_div_(Tensor &x, float value) {
  RV_CHECK(x.dtype() == DType::kFloat16) << "scalar_div_ on hip is defined for fp16 (model_forward.cpp:173-175)";
  FRHIP_CHECK(frhip_scalar_div_f16(x.data_ptr(), value, static_cast<size_t>(x.numel()), stream()));
  return x;
}

Tensor layernorm(const Tensor &x, const Tensor &weight, const Tensor &bias) {
  RV_CHECK(x.sizes().size() <= 2);
  RV_CHECK(x.dtype() == weight.dtype() && x.dtype() == bias.dtype());
  const int rows = x.sizes().size() == 1 ? 1 : static_cast<int>(x.size(0));
  const int cols = static_cast<int>(x.size(-1));
  Tensor y = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_layernorm(x.data_ptr(), weight.data_ptr(), bias.data_ptr(), y.data_ptr(), rows, cols,
                              to_frhip_dtype(x.dtype()), stream()));
  return y;
}

Tensor groupnorm(const Tensor &x, int num_groups, const Tensor &weight, const Tensor &bias) {
  RV_CHECK(x.sizes().size() <= 2);
  RV_CHECK(x.dtype() == DType::kFloat32 && weight.dtype() == DType::kFloat32 && bias.dtype() == DType::kFloat32)
      << "groupnorm on hip runs on fp32 (the dtype the RWKV-5 path gives it)";
  const int rows = x.sizes().size() == 1 ? 1 : static_cast<int>(x.size(0));
  const int cols = static_cast<int>(x.size(-1));
  Tensor y = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_groupnorm_f32(x.data_ptr<float>(), num_groups, weight.data_ptr<float>(), bias.data_ptr<float>(),
                                  y.data_ptr<float>(), rows, cols, stream()));
  return y;
}

// matmul (reference: kernels/cuda/matmul.cpp:123-146).  Vector x matrix runs the
// row-streaming kernel; output dtype = activation dtype.
Tensor matmul(const Tensor &a, const Tensor &b) {
  RV_CHECK(a.device() == b.device());
  RV_CHECK(a.dtype() == DType::kFloat16) << "matmul on hip: activations are fp16";
  RV_CHECK((a.sizes().size() == 1 || a.sizes().size() == 2) && b.sizes().size() == 2)
      << "matmul on hip: [K] x [K, N] or [T, K] x [K, N]";
  RV_CHECK(a.size(-1) == b.size(0)) << "matmul: " << shape_str(a.shape()) << " x " << shape_str(b.shape());
  frhip_weight tmp_desc;
  Tensor tmp;
  const frhip_weight *w = weight_of(b, tmp_desc, tmp, a.sizes().size() == 2 ? static_cast<int>(a.size(0)) : 1);
  if (a.sizes().size() == 2) {  // matrix x matrix (matmul.cpp:110-121): the MFMA product
    const int T = static_cast<int>(a.size(0));
    Tensor c = Tensor::Empty({a.size(0), b.size(1)}, a.dtype(), Device::kHIP);
    FRHIP_CHECK(frhip_gemm(a.data_ptr(), w, c.data_ptr(), T, FRHIP_F16, stream()));
    return c;
  }
  Tensor c = Tensor::Empty({b.size(1)}, a.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_gemv(a.data_ptr(), w, c.data_ptr(), FRHIP_F16, stream()));
  return c;
}

// vgather (reference: kernels/default/gather_ops.cpp:46-89): rows are copied device to
// device.  When the rows are views into one table (as this backend's init_model makes
// them) the copies are contiguous slices of that table.
Tensor vgather(const std::vector<Tensor> &x, const std::vector<int> &idx) {
  Shape shape{static_cast<LengthType>(idx.size())};
  shape.insert(shape.end(), x[0].shape().begin(), x[0].shape().end());
  Tensor out = Tensor::Empty(shape, x[0].dtype(), Device::kHIP);
  const size_t row = x[0].nbytes();
  char *dst = static_cast<char *>(out.data_ptr());
  for (size_t i = 0; i < idx.size(); i++) {
    RV_CHECK(idx[i] >= 0 && static_cast<size_t>(idx[i]) < x.size());
    FRHIP_CHECK(frhip_memcpy_async(dst + i * row, x[idx[i]].data_ptr(), row, FRHIP_D2D, stream()));
  }
  return out;
}

// slice (reference: kernels/cuda/slice.cu:38-136).  Range semantics as there: (0,0,0) is the whole
// dimension, negative start / end count from the end, output extent (end - start) / interval.
// Leading-dimension ranges of a contiguous tensor (the last row that model_forward_seq.cpp:171
// takes, all rows but the last of a token shift) are views into the source, no copy and no launch.
Tensor slice(const Tensor &x, const std::vector<Range> &ranges) {
  RV_CHECK(x.sizes().size() == ranges.size() && !ranges.empty() && ranges.size() <= 4);
  const int nd = static_cast<int>(ranges.size());
  int src[4], start[4], interval[4], dst[4];
  Shape out_shape;
  bool inner_whole = true;  // every dimension after the first is taken whole
  for (int i = 0; i < nd; i++) {
    const int dim = static_cast<int>(x.size(i));
    int st = ranges[i].start, iv = ranges[i].interval, en = ranges[i].end;
    if (st == 0 && iv == 0 && en == 0) {
      en = dim;
      iv = 1;
    }
    if (st < 0) st += dim;
    if (en < 0) en += dim;
    RV_CHECK(iv > 0);
    RV_CHECK(st >= 0 && st <= en && en <= dim);
    src[i] = dim;
    start[i] = st;
    interval[i] = iv;
    dst[i] = (en - st) / iv;
    out_shape.push_back(dst[i]);
    if (i > 0 && !(st == 0 && iv == 1 && en == dim)) inner_whole = false;
  }
  if (inner_whole && interval[0] == 1 && dst[0] > 0) {
    const size_t row = x.nbytes() / static_cast<size_t>(src[0]);
    return Tensor::SubView(x, static_cast<size_t>(start[0]) * row, out_shape);
  }
  Tensor out = Tensor::Empty(out_shape, x.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_slice(x.data_ptr(), out.data_ptr(), nd, src, start, interval, dst, x.elem_size(), stream()));
  return out;
}

// cat (reference: kernels/cuda/cat.cu:57-111).
Tensor cat(const Tensor &a, const Tensor &b, int dim) {
  RV_CHECK(a.sizes().size() == b.sizes().size());
  RV_CHECK(a.dtype() == b.dtype());
  RV_CHECK(a.device() == b.device());
  const int nd = static_cast<int>(a.sizes().size());
  if (dim < 0) dim += nd;
  RV_CHECK(dim >= 0 && dim < nd);
  size_t left = 1, right = 1;
  Shape out_shape;
  for (int i = 0; i < nd; i++) {
    if (i != dim) RV_CHECK(a.size(i) == b.size(i));
    if (i < dim) left *= static_cast<size_t>(a.size(i));
    if (i > dim) right *= static_cast<size_t>(a.size(i));
    out_shape.push_back(i == dim ? a.size(i) + b.size(i) : a.size(i));
  }
  Tensor out = Tensor::Empty(out_shape, a.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_cat(a.data_ptr(), b.data_ptr(), out.data_ptr(), left, static_cast<size_t>(a.size(dim)),
                        static_cast<size_t>(b.size(dim)), right, a.elem_size(), stream()));
  return out;
}

// transpose (reference: kernels/cuda/transpose.cu:91-103).
Tensor transpose(const Tensor &x, int dim_a, int dim_b) {
  const int nd = static_cast<int>(x.sizes().size());
  RV_CHECK(nd >= 2 && nd <= 4);
  if (dim_a < 0) dim_a += nd;
  if (dim_b < 0) dim_b += nd;
  RV_CHECK(dim_a >= 0 && dim_b >= 0);
  RV_CHECK(dim_a < nd && dim_b < nd);
  Shape out_shape = x.shape();
  std::swap(out_shape[dim_a], out_shape[dim_b]);
  int shape[4];
  for (int i = 0; i < nd; i++) shape[i] = static_cast<int>(x.size(i));
  Tensor out = Tensor::Empty(out_shape, x.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_transpose(x.data_ptr(), out.data_ptr(), nd, shape, dim_a, dim_b, x.elem_size(), stream()));
  return out;
}

// silu (reference: kernels/cuda/activations/silu.cu:38-57; the arithmetic is InplaceSiLU's,
// kernels/cuda/att.cu:145-152 -- the standalone reference kernel is not SiLU).
Tensor silu(const Tensor &x) {
  RV_CHECK(x.dtype() == DType::kFloat16 || x.dtype() == DType::kFloat32);
  Tensor y = Tensor::Empty(x.shape(), x.dtype(), Device::kHIP);
  FRHIP_CHECK(frhip_silu(x.data_ptr(), y.data_ptr(), to_frhip_dtype(x.dtype()), static_cast<size_t>(x.numel()), stream()));
  return y;
}

// att, RWKV-4 one token (reference: kernels/cuda/att.cu:337-359).
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor>
att(const Tensor &x, const Tensor &sx, const Tensor &aa, const Tensor &bb, const Tensor &pp, const Tensor &ln_w,
    const Tensor &ln_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix, const Tensor &t_decay,
    const Tensor &t_first, const Tensor &kw, const Tensor &vw, const Tensor &rw, const Tensor &ow) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 1);
  const int C = static_cast<int>(x.size(0));
  frhip_weight d[4];
  Tensor tmp[4];
  const frhip_weight *w[4] = {weight_of(kw, d[0], tmp[0]), weight_of(vw, d[1], tmp[1]), weight_of(rw, d[2], tmp[2]),
                              weight_of(ow, d[3], tmp[3])};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor t1 = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor t2 = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor p = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = workspace(C, 16);
  FRHIP_CHECK(frhip_att_one_v4(C, x.data_ptr(), sx.data_ptr(), aa.data_ptr<float>(), bb.data_ptr<float>(),
                               pp.data_ptr<float>(), ln_w.data_ptr(), ln_b.data_ptr(), k_mix.data_ptr(),
                               v_mix.data_ptr(), r_mix.data_ptr(), t_decay.data_ptr<float>(),
                               t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], x_out.data_ptr(), xx.data_ptr(),
                               t1.data_ptr<float>(), t2.data_ptr<float>(), p.data_ptr<float>(), ws.data_ptr(),
                               stream()));
  return {x_out, xx, t1, t2, p};
}

// ffn, one token (reference: kernels/cuda/ffn.cu:89-110).
std::tuple<Tensor, Tensor> ffn(const Tensor &x, const Tensor &sx, const Tensor &ln_w, const Tensor &ln_b,
                               const Tensor &k_mix, const Tensor &r_mix, const Tensor &kw, const Tensor &vw,
                               const Tensor &rw) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 1);
  const int C = static_cast<int>(x.size(0));
  const int F = static_cast<int>(kw.size(1));
  frhip_weight d[3];
  Tensor tmp[3];
  const frhip_weight *w[3] = {weight_of(kw, d[0], tmp[0]), weight_of(vw, d[1], tmp[1]), weight_of(rw, d[2], tmp[2])};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor ws = workspace(C, F);
  FRHIP_CHECK(frhip_ffn_one(C, F, x.data_ptr(), sx.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), k_mix.data_ptr(),
                            r_mix.data_ptr(), w[0], w[1], w[2], x_out.data_ptr(), xx.data_ptr(), 0, ws.data_ptr(),
                            stream()));
  return {x_out, xx};
}

// att_one_v5_1, RWKV-5.1/5.2 one token (reference: kernels/cuda/att.cu:393-425).
std::tuple<Tensor, Tensor, Tensor>
att_one_v5_1(const Tensor &x, const Tensor &sx, const Tensor &s, const Tensor &ln_w, const Tensor &ln_b,
             const Tensor &lx_w, const Tensor &lx_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix,
             const Tensor &g_mix, const Tensor &t_decay, const Tensor &t_first, const Tensor &kw, const Tensor &vw,
             const Tensor &rw, const Tensor &gw, const Tensor &ow) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 1);
  const int C = static_cast<int>(x.size(0));
  const int H = static_cast<int>(t_decay.size(0));
  frhip_weight d[5];
  Tensor tmp[5];
  const frhip_weight *w[5] = {weight_of(kw, d[0], tmp[0]), weight_of(vw, d[1], tmp[1]), weight_of(rw, d[2], tmp[2]),
                              weight_of(gw, d[3], tmp[3]), weight_of(ow, d[4], tmp[4])};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor s_out = Tensor::Empty(s.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = workspace(C, 16);
  FRHIP_CHECK(frhip_att_one_v5_1(C, H, x.data_ptr(), sx.data_ptr(), s.data_ptr<float>(), ln_w.data_ptr(),
                                 ln_b.data_ptr(), lx_w.data_ptr<float>(), lx_b.data_ptr<float>(), k_mix.data_ptr(),
                                 v_mix.data_ptr(), r_mix.data_ptr(), g_mix.data_ptr(), t_decay.data_ptr<float>(),
                                 t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], w[4], x_out.data_ptr(),
                                 xx.data_ptr(), s_out.data_ptr<float>(), ws.data_ptr(), stream()));
  return {x_out, xx, s_out};
}

// att_one_v5, RWKV-5.0 one token (reference: kernels/cuda/att.cu:362-391).  t_decay and
// t_first hold one value per head ([H] or [H,1,1]).
std::tuple<Tensor, Tensor, Tensor>
att_one_v5(const Tensor &x, const Tensor &sx, const Tensor &s, const Tensor &ln_w, const Tensor &ln_b,
           const Tensor &lx_w, const Tensor &lx_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix,
           const Tensor &t_decay, const Tensor &t_first, const Tensor &kw, const Tensor &vw, const Tensor &rw,
           const Tensor &ow) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 1);
  const int C = static_cast<int>(x.size(0));
  const int H = static_cast<int>(t_decay.size(0));
  RV_CHECK(t_decay.numel() == H && t_first.numel() == H) << "att_one_v5: time_decay/time_first must hold one value per head";
  frhip_weight d[4];
  Tensor tmp[4];
  const frhip_weight *w[4] = {weight_of(kw, d[0], tmp[0]), weight_of(vw, d[1], tmp[1]), weight_of(rw, d[2], tmp[2]),
                              weight_of(ow, d[3], tmp[3])};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor s_out = Tensor::Empty(s.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = workspace(C, 16);
  FRHIP_CHECK(frhip_att_one_v5(C, H, x.data_ptr(), sx.data_ptr(), s.data_ptr<float>(), ln_w.data_ptr(),
                               ln_b.data_ptr(), lx_w.data_ptr<float>(), lx_b.data_ptr<float>(), k_mix.data_ptr(),
                               v_mix.data_ptr(), r_mix.data_ptr(), t_decay.data_ptr<float>(),
                               t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], x_out.data_ptr(), xx.data_ptr(),
                               s_out.data_ptr<float>(), ws.data_ptr(), stream()));
  return {x_out, xx, s_out};
}

static Tensor seq_workspace(int T, int C, int F) {
  return Tensor::Empty({static_cast<LengthType>(frhip_seq_workspace_bytes(T, C, F))}, DType::kInt8, Device::kHIP);
}

// ffn_seq (reference: kernels/cuda/ffn_seq.cu:89-109).  x [T, C]; returns (x_out [T, C], LN(x)[T-1]).
// `div2`: the result rows are halved in binary16 after the residual, as scalar_div_(x_out, 2) would
// (model_forward_seq.cpp:163-165 does that as an operator of its own every sixth layer).
std::tuple<Tensor, Tensor> ffn_seq_div2(const Tensor &x, const Tensor &sx, const Tensor &ln_w, const Tensor &ln_b,
                                        const Tensor &k_mix, const Tensor &r_mix, const Tensor &kw, const Tensor &vw,
                                        const Tensor &rw, bool div2) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 2);
  const int T = static_cast<int>(x.size(0)), C = static_cast<int>(x.size(1)), F = static_cast<int>(kw.size(1));
  frhip_weight d[3];
  Tensor tmp[3];
  const frhip_weight *w[3] = {weight_of(kw, d[0], tmp[0], T), weight_of(vw, d[1], tmp[1], T), weight_of(rw, d[2], tmp[2], T)};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty({C}, x.dtype(), Device::kHIP);
  Tensor ws = seq_workspace(T, C, F);
  FRHIP_CHECK(frhip_ffn_seq(T, C, F, x.data_ptr(), sx.data_ptr(), ln_w.data_ptr(), ln_b.data_ptr(), k_mix.data_ptr(),
                            r_mix.data_ptr(), w[0], w[1], w[2], x_out.data_ptr(), xx.data_ptr(), div2 ? 1 : 0,
                            ws.data_ptr(), stream()));
  return {x_out, xx};
}

std::tuple<Tensor, Tensor> ffn_seq(const Tensor &x, const Tensor &sx, const Tensor &ln_w, const Tensor &ln_b,
                                   const Tensor &k_mix, const Tensor &r_mix, const Tensor &kw, const Tensor &vw,
                                   const Tensor &rw) {
  return ffn_seq_div2(x, sx, ln_w, ln_b, k_mix, r_mix, kw, vw, rw, false);
}

// att_seq, RWKV-4 (no counterpart upstream: kernels/default/model_forward_seq.cpp:111-112 throws).
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor>
att_seq(const Tensor &x, const Tensor &sx, const Tensor &aa, const Tensor &bb, const Tensor &pp, const Tensor &ln_w,
        const Tensor &ln_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix, const Tensor &t_decay,
        const Tensor &t_first, const Tensor &kw, const Tensor &vw, const Tensor &rw, const Tensor &ow) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 2);
  const int T = static_cast<int>(x.size(0)), C = static_cast<int>(x.size(1));
  frhip_weight d[4];
  Tensor tmp[4];
  const frhip_weight *w[4] = {weight_of(kw, d[0], tmp[0], T), weight_of(vw, d[1], tmp[1], T), weight_of(rw, d[2], tmp[2], T),
                              weight_of(ow, d[3], tmp[3], T)};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty({C}, x.dtype(), Device::kHIP);
  Tensor t1 = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor t2 = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor p = Tensor::Empty(aa.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = seq_workspace(T, C, 64);
  FRHIP_CHECK(frhip_att_seq_v4(T, C, x.data_ptr(), sx.data_ptr(), aa.data_ptr<float>(), bb.data_ptr<float>(),
                               pp.data_ptr<float>(), ln_w.data_ptr(), ln_b.data_ptr(), k_mix.data_ptr(),
                               v_mix.data_ptr(), r_mix.data_ptr(), t_decay.data_ptr<float>(),
                               t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], x_out.data_ptr(), xx.data_ptr(),
                               t1.data_ptr<float>(), t2.data_ptr<float>(), p.data_ptr<float>(), ws.data_ptr(),
                               stream()));
  return {x_out, xx, t1, t2, p};
}

// att_seq_v5_2 (reference: kernels/cuda/att_seq.cu:464-493).
std::tuple<Tensor, Tensor, Tensor>
att_seq_v5_2(const Tensor &x, const Tensor &sx, const Tensor &s, const Tensor &ln_w, const Tensor &ln_b,
             const Tensor &lx_w, const Tensor &lx_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix,
             const Tensor &g_mix, const Tensor &t_decay, const Tensor &t_first, const Tensor &kw, const Tensor &vw,
             const Tensor &rw, const Tensor &gw, const Tensor &ow, int n_att) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 2);
  const int T = static_cast<int>(x.size(0)), C = static_cast<int>(x.size(1));
  RV_CHECK(n_att == C) << "att_seq_v5_2 on hip: n_att must equal n_embd";
  const int H = static_cast<int>(t_decay.size(0));
  frhip_weight d[5];
  Tensor tmp[5];
  const frhip_weight *w[5] = {weight_of(kw, d[0], tmp[0], T), weight_of(vw, d[1], tmp[1], T), weight_of(rw, d[2], tmp[2], T),
                              weight_of(gw, d[3], tmp[3], T), weight_of(ow, d[4], tmp[4], T)};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty({C}, x.dtype(), Device::kHIP);
  Tensor s_out = Tensor::Empty(s.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = seq_workspace(T, C, 64);
  FRHIP_CHECK(frhip_att_seq_v5_2(T, C, H, x.data_ptr(), sx.data_ptr(), s.data_ptr<float>(), ln_w.data_ptr(),
                                 ln_b.data_ptr(), lx_w.data_ptr<float>(), lx_b.data_ptr<float>(), k_mix.data_ptr(),
                                 v_mix.data_ptr(), r_mix.data_ptr(), g_mix.data_ptr(), t_decay.data_ptr<float>(),
                                 t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], w[4], x_out.data_ptr(),
                                 xx.data_ptr(), s_out.data_ptr<float>(), ws.data_ptr(), stream()));
  return {x_out, xx, s_out};
}

// att_seq_v5, RWKV-5.0 (reference: kernels/cuda/att_seq.cu:425-462).
std::tuple<Tensor, Tensor, Tensor>
att_seq_v5(const Tensor &x, const Tensor &sx, const Tensor &s, const Tensor &ln_w, const Tensor &ln_b,
           const Tensor &lx_w, const Tensor &lx_b, const Tensor &k_mix, const Tensor &v_mix, const Tensor &r_mix,
           const Tensor &t_decay, const Tensor &t_first, const Tensor &kw, const Tensor &vw, const Tensor &rw,
           const Tensor &ow) {
  RV_CHECK(x.dtype() == DType::kFloat16 && x.sizes().size() == 2);
  const int T = static_cast<int>(x.size(0)), C = static_cast<int>(x.size(1));
  const int H = static_cast<int>(t_decay.size(0));
  RV_CHECK(t_decay.numel() == H && t_first.numel() == H) << "att_seq_v5: time_decay/time_first must hold one value per head";
  frhip_weight d[4];
  Tensor tmp[4];
  const frhip_weight *w[4] = {weight_of(kw, d[0], tmp[0], T), weight_of(vw, d[1], tmp[1], T), weight_of(rw, d[2], tmp[2], T),
                              weight_of(ow, d[3], tmp[3], T)};
  Tensor x_out = Tensor::Empty(x.sizes(), x.dtype(), Device::kHIP);
  Tensor xx = Tensor::Empty({C}, x.dtype(), Device::kHIP);
  Tensor s_out = Tensor::Empty(s.sizes(), DType::kFloat32, Device::kHIP);
  Tensor ws = seq_workspace(T, C, 64);
  FRHIP_CHECK(frhip_att_seq_v5(T, C, H, x.data_ptr(), sx.data_ptr(), s.data_ptr<float>(), ln_w.data_ptr(),
                               ln_b.data_ptr(), lx_w.data_ptr<float>(), lx_b.data_ptr<float>(), k_mix.data_ptr(),
                               v_mix.data_ptr(), r_mix.data_ptr(), t_decay.data_ptr<float>(),
                               t_first.data_ptr<float>(), w[0], w[1], w[2], w[3], x_out.data_ptr(), xx.data_ptr(),
                               s_out.data_ptr<float>(), ws.data_ptr(), stream()));
  return {x_out, xx, s_out};
}

KernelRegister fill_reg("fill_", Device::kHIP, fill_);
KernelRegister cast_reg("cast_dtype", Device::kHIP, cast_dtype);
KernelRegister scalar_div_reg("scalar_div_", Device::kHIP, scalar_div_);
KernelRegister layernorm_reg("layernorm", Device::kHIP, layernorm);
KernelRegister groupnorm_reg("groupnorm", Device::kHIP, groupnorm);
KernelRegister matmul_reg("matmul", Device::kHIP, matmul);
KernelRegister vgather_reg("vgather", Device::kHIP, vgather);
KernelRegister slice_reg("slice", Device::kHIP, slice);
KernelRegister cat_reg("cat", Device::kHIP, cat);
KernelRegister transpose_reg("transpose", Device::kHIP, transpose);
KernelRegister silu_reg("silu", Device::kHIP, silu);
KernelRegister att_reg("att", Device::kHIP, att);
KernelRegister ffn_reg("ffn", Device::kHIP, ffn);
KernelRegister ffn_seq_reg("ffn_seq", Device::kHIP, ffn_seq);
KernelRegister att_seq_reg("att_seq", Device::kHIP, att_seq);
KernelRegister att_seq_v5_2_reg("att_seq_v5_2", Device::kHIP, att_seq_v5_2);
KernelRegister att_one_v5_1_reg("att_one_v5_1", Device::kHIP, att_one_v5_1);
KernelRegister att_one_v5_reg("att_one_v5", Device::kHIP, att_one_v5);
KernelRegister att_seq_v5_reg("att_seq_v5", Device::kHIP, att_seq_v5);

}  // namespace hip
}  // namespace rwkv
