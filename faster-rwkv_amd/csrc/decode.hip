// One-token (batch-1 decode) kernels for gfx950.
//
// The decode step of RWKV is a chain of matrix-vector products separated by cheap
// elementwise work; each product streams its weight matrix from HBM exactly once,
// so the whole step is bound by HBM bandwidth.  The kernels here are organised
// around that:
//   * weights are output-major ([N][K]); a wavefront takes whole rows, each lane
//     loads 16 contiguous bytes per row chunk, products accumulate in fp32 and are
//     reduced across lanes with DPP adds.  No partial sums ever leave the wave, so
//     every elementwise epilogue (sigmoid, WKV update, relu^2, residual) runs in
//     the lane that owns the output and is fused into the same launch;
//   * the layernorm + token-shift mix that precedes a product is recomputed by
//     every workgroup into LDS (the activation vector is a few KB and L2-resident),
//     which removes the separate launches the reference makes for them
//     (kernels/cuda/att.cu:183-188, ffn.cu:66-75);
//   * independent products share a launch (key/value/receptance of att; receptance
//     and key of ffn) so that a launch moves tens of MB.
// One RWKV-4 layer is four launches; the reference issues seventeen
// (kernels/cuda/att.cu:182-217, ffn.cu:62-87).
#include "device_utils.h"
#include "frhip_internal.h"

#pragma clang fp contract(off)

namespace frhip {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;

struct WMat {
  const unsigned char* data;
  const h1 *mx, *rx, *my, *ry;
  int K, N;
};

static WMat to_wmat(const frhip_weight* w) {
  WMat m;
  m.data = static_cast<const unsigned char*>(w->data);
  m.mx = static_cast<const h1*>(w->mx);
  m.rx = static_cast<const h1*>(w->rx);
  m.my = static_cast<const h1*>(w->my);
  m.ry = static_cast<const h1*>(w->ry);
  m.K = w->K;
  m.N = w->N;
  return m;
}

// ---------------------------------------------------------------------------
// layernorm of a [C] vector by a whole workgroup; thread t owns elements
// [8t, 8t+8).  Requires C % 8 == 0 and C <= 8 * kThreads.
// kernels/cuda/layer_norm.cu:60-69: normalise in fp32, round to half, multiply by
// gamma in half, add beta in half.
// ---------------------------------------------------------------------------
struct LnOut {
  h8 xx;
  bool active;
};

__device__ __forceinline__ LnOut ln_block(const h1* x, const h1* gamma, const h1* beta, int C, float* red) {
  const int e0 = threadIdx.x * 8;
  LnOut o;
  o.active = e0 < C;
  float xf[8];
  float s = 0.f;
  if (o.active) {
    h8 xv = *reinterpret_cast<const h8*>(x + e0);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      xf[i] = (float)xv[i];
      s += xf[i];
    }
  }
  const float mean = block_sum<kWaves>(s, red) / (float)C;
  float q = 0.f;
  if (o.active) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      float d = xf[i] - mean;
      q += d * d;
    }
  }
  float var = block_sum<kWaves>(q, red) / (float)C;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
  if (o.active) {
    h8 g = *reinterpret_cast<const h8*>(gamma + e0);
    h8 b = *reinterpret_cast<const h8*>(beta + e0);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      h1 n = (h1)((xf[i] - mean) * inv);
      o.xx[i] = (n * g[i]) + b[i];
    }
  }
  return o;
}

__device__ __forceinline__ h8 mix8(h8 xx, h8 sx, h8 m) {
  h8 o;
#pragma unroll
  for (int i = 0; i < 8; i++) o[i] = mix1(xx[i], sx[i], m[i]);
  return o;
}

// Rows [r0, r1) of one matrix against one staged vector, R rows in flight per
// wave; lane j (j < R) receives the finished sum of row n+j and runs the epilogue.
template <int R, bool U8, class Epi>
__device__ __forceinline__ void gemv_rows(const WMat& m, const XVec& xv, int r0, int r1, int lane, Epi epi) {
  const size_t row_bytes = U8 ? (size_t)m.K : 2 * (size_t)m.K;
  for (int n = r0; n < r1; n += R) {
    const void* rows[R];
    XVec xvs[R];
    RowQ rq[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      int nn = n + r < r1 ? n + r : r1 - 1;  // clamp: surplus slots re-read the last row
      rows[r] = m.data + (size_t)nn * row_bytes;
      xvs[r] = xv;
      if constexpr (U8) {
        rq[r].c255 = dequant_c255(m.rx[nn]);
        rq[r].mx = m.mx[nn];
      }
    }
    float acc[R];
    dot_rows<R, U8>(rows, xvs, rq, m.K, lane, acc);
    float mine = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
      float t = wave_sum(acc[r]);
      if (lane == r) mine = t;
    }
    if (lane < R && n + lane < r1) epi(n + lane, mine);
  }
}

// Even split of `total` items over `parts`: part i gets [lo, hi).
__device__ __forceinline__ void split_even(int total, int parts, int i, int& lo, int& hi) {
  lo = (int)(((long long)total * i) / parts);
  hi = (int)(((long long)total * (i + 1)) / parts);
}

// ===========================================================================
// att, front half:  LN -> mix -> k,v,r products -> sigmoid -> WKV-4 update
//                   -> r * wkv                    (kernels/cuda/att.cu:183-211)
// ===========================================================================
struct AttFrontV4 {
  int C;
  const h1 *x, *sx, *ln_w, *ln_b, *mk, *mv, *mr;
  const float *aa, *bb, *pp, *td, *tf;
  WMat kw, vw, rw;
  h1 *xx_out, *rwkv_out;
  float *aa_out, *bb_out, *pp_out;
};

template <bool U8>
__global__ __launch_bounds__(kThreads) void att_front_v4_kernel(AttFrontV4 a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[kWaves];
  const int C = a.C;
  h1* kx = reinterpret_cast<h1*>(smem);
  h1* vx = kx + C;
  h1* rx = vx + C;
  h1* qv = rx + C;  // uint8 only: ry,my of kw ; ry,my of vw ; ry,my of rw

  LnOut ln = ln_block(a.x, a.ln_w, a.ln_b, C, red);
  if (ln.active) {
    const int e0 = threadIdx.x * 8;
    h8 sx = *reinterpret_cast<const h8*>(a.sx + e0);
    const int pos = stage_pos<U8>(threadIdx.x, C);
    reinterpret_cast<h8*>(kx)[pos] = mix8(ln.xx, sx, *reinterpret_cast<const h8*>(a.mk + e0));
    reinterpret_cast<h8*>(vx)[pos] = mix8(ln.xx, sx, *reinterpret_cast<const h8*>(a.mv + e0));
    reinterpret_cast<h8*>(rx)[pos] = mix8(ln.xx, sx, *reinterpret_cast<const h8*>(a.mr + e0));
    if (blockIdx.x == 0) *reinterpret_cast<h8*>(a.xx_out + e0) = ln.xx;
  }
  if constexpr (U8) {
    stage_vec<true>(qv + 0 * C, a.kw.ry, C);
    stage_vec<true>(qv + 1 * C, a.kw.my, C);
    stage_vec<true>(qv + 2 * C, a.vw.ry, C);
    stage_vec<true>(qv + 3 * C, a.vw.my, C);
    stage_vec<true>(qv + 4 * C, a.rw.ry, C);
    stage_vec<true>(qv + 5 * C, a.rw.my, C);
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int gw = blockIdx.x * kWaves + threadIdx.x / kWave;
  int c0, c1;
  split_even(C, gridDim.x * kWaves, gw, c0, c1);
  const size_t row_bytes = U8 ? (size_t)C : 2 * (size_t)C;
  for (int n = c0; n < c1; n++) {
    const void* rows[3] = {a.kw.data + n * row_bytes, a.vw.data + n * row_bytes, a.rw.data + n * row_bytes};
    XVec xv[3] = {{kx, qv + 0 * C, qv + 1 * C}, {vx, qv + 2 * C, qv + 3 * C}, {rx, qv + 4 * C, qv + 5 * C}};
    RowQ rq[3];
    if constexpr (U8) {
      rq[0] = {dequant_c255(a.kw.rx[n]), a.kw.mx[n]};
      rq[1] = {dequant_c255(a.vw.rx[n]), a.vw.mx[n]};
      rq[2] = {dequant_c255(a.rw.rx[n]), a.rw.mx[n]};
    }
    float acc[3];
    dot_rows<3, U8>(rows, xv, rq, C, lane, acc);
    const float k = wave_sum(acc[0]);
    const float v = wave_sum(acc[1]);
    const float rr = wave_sum(acc[2]);
    if (lane == 0) {
      // kernels/cuda/att.cu:30-62 (WkvForwardOne), r already passed through sigmoid (:203)
      const h1 r = sigmoid_h((h1)rr);
      float ww = a.tf[n] + k;
      const float pp_ = a.pp[n];
      float p_ = (pp_ > ww) ? pp_ : ww;
      float e1 = expf(pp_ - p_);
      float e2 = expf(ww - p_);
      const float aa_ = a.aa[n], bb_ = a.bb[n];
      const float wkv = (e1 * aa_ + e2 * v) / (e1 * bb_ + e2);
      a.rwkv_out[n] = r * (h1)wkv;
      ww = a.td[n] + pp_;
      p_ = (ww > k) ? ww : k;
      e1 = expf(ww - p_);
      e2 = expf(k - p_);
      a.aa_out[n] = e1 * aa_ + e2 * v;
      a.bb_out[n] = e1 * bb_ + e2;
      a.pp_out[n] = p_;
    }
  }
}

// ===========================================================================
// Generic "stage a vector, stream rows, epilogue per output" kernels
// ===========================================================================
// att, back half: out = rwkv . Wo ; x_out = x + out     (att.cu:213-215)
struct AttOutV4 {
  int C;
  const h1 *rwkv, *x;
  WMat ow;
  h1* x_out;
};

template <int R, bool U8>
__global__ __launch_bounds__(kThreads) void att_out_kernel(AttOutV4 a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = a.ow.K;
  h1* xs = reinterpret_cast<h1*>(smem);
  stage_vec<U8>(xs, a.rwkv, K);
  if constexpr (U8) {
    stage_vec<true>(xs + K, a.ow.ry, K);
    stage_vec<true>(xs + 2 * K, a.ow.my, K);
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  int r0, r1;
  split_even(a.ow.N, gridDim.x * kWaves, blockIdx.x * kWaves + threadIdx.x / kWave, r0, r1);
  XVec xv = {xs, xs + K, xs + 2 * K};
  gemv_rows<R, U8>(a.ow, xv, r0, r1, lane, [&](int n, float sum) { a.x_out[n] = a.x[n] + (h1)sum; });
}

// ffn, front half: LN -> mix -> r = sigmoid(rx.Wr) ; vx = relu(kx.Wk)^2   (ffn.cu:66-81)
struct FfnFront {
  int C, F;
  const h1 *x, *sx, *ln_w, *ln_b, *mk, *mr;
  WMat kw, rw;
  h1 *xx_out, *r_out, *vx_out;
};

template <int R, bool U8>
__global__ __launch_bounds__(kThreads) void ffn_front_kernel(FfnFront a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[kWaves];
  const int C = a.C, F = a.F;
  h1* kx = reinterpret_cast<h1*>(smem);
  h1* rx = kx + C;
  h1* qv = rx + C;  // uint8 only: ry,my of rw ; ry,my of kw  (all [C])
  LnOut ln = ln_block(a.x, a.ln_w, a.ln_b, C, red);
  if (ln.active) {
    const int e0 = threadIdx.x * 8;
    h8 sx = *reinterpret_cast<const h8*>(a.sx + e0);
    const int pos = stage_pos<U8>(threadIdx.x, C);
    reinterpret_cast<h8*>(kx)[pos] = mix8(ln.xx, sx, *reinterpret_cast<const h8*>(a.mk + e0));
    reinterpret_cast<h8*>(rx)[pos] = mix8(ln.xx, sx, *reinterpret_cast<const h8*>(a.mr + e0));
    if (blockIdx.x == 0) *reinterpret_cast<h8*>(a.xx_out + e0) = ln.xx;
  }
  if constexpr (U8) {
    stage_vec<true>(qv + 0 * C, a.rw.ry, C);
    stage_vec<true>(qv + 1 * C, a.rw.my, C);
    stage_vec<true>(qv + 2 * C, a.kw.ry, C);
    stage_vec<true>(qv + 3 * C, a.kw.my, C);
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  int g0, g1;  // rows [0,C) are receptance rows, [C, C+F) key rows
  split_even(C + F, gridDim.x * kWaves, blockIdx.x * kWaves + threadIdx.x / kWave, g0, g1);
  if (g0 < C) {
    XVec xv = {rx, qv + 0 * C, qv + 1 * C};
    gemv_rows<R, U8>(a.rw, xv, g0, g1 < C ? g1 : C, lane,
                     [&](int n, float sum) { a.r_out[n] = sigmoid_h((h1)sum); });
  }
  if (g1 > C) {
    XVec xv = {kx, qv + 2 * C, qv + 3 * C};
    gemv_rows<R, U8>(a.kw, xv, (g0 > C ? g0 : C) - C, g1 - C, lane, [&](int n, float sum) {
      h1 t = (h1)sum;  // ffn.cu:41-51
      a.vx_out[n] = (t > (h1)0.0f) ? (t * t) : (h1)0.0f;
    });
  }
}

// ffn, back half: out = vx.Wv ; x_out = fma(out, r, x) [; x_out /= 2]   (ffn.cu:82-85)
struct FfnOut {
  int C, F;
  const h1 *vx, *r, *x;
  WMat vw;
  h1* x_out;
  int div2;
};

template <int R, bool U8>
__global__ __launch_bounds__(kThreads) void ffn_out_kernel(FfnOut a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = a.vw.K;
  h1* xs = reinterpret_cast<h1*>(smem);
  stage_vec<U8>(xs, a.vx, K);
  if constexpr (U8) {
    stage_vec<true>(xs + K, a.vw.ry, K);
    stage_vec<true>(xs + 2 * K, a.vw.my, K);
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  int r0, r1;
  split_even(a.vw.N, gridDim.x * kWaves, blockIdx.x * kWaves + threadIdx.x / kWave, r0, r1);
  XVec xv = {xs, xs + K, xs + 2 * K};
  gemv_rows<R, U8>(a.vw, xv, r0, r1, lane, [&](int n, float sum) {
    h1 o = __builtin_fmaf16((h1)sum, a.r[n], a.x[n]);       // __hfma, one rounding
    if (a.div2) o = o / (h1)2.0f;                           // model_forward.cpp:173-175
    a.x_out[n] = o;
  });
}

// head: LN(ln_out) -> x.Whead -> half -> fp32   (model_forward.cpp:180-188)
struct Head {
  int C;
  const h1 *x, *ln_w, *ln_b;
  WMat hw;
  float* logits;
};

template <int R, bool U8>
__global__ __launch_bounds__(kThreads) void head_kernel(Head a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[kWaves];
  const int C = a.C;
  h1* xs = reinterpret_cast<h1*>(smem);
  LnOut ln = ln_block(a.x, a.ln_w, a.ln_b, C, red);
  if (ln.active) reinterpret_cast<h8*>(xs)[stage_pos<U8>(threadIdx.x, C)] = ln.xx;
  if constexpr (U8) {
    stage_vec<true>(xs + C, a.hw.ry, C);
    stage_vec<true>(xs + 2 * C, a.hw.my, C);
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  int r0, r1;
  split_even(a.hw.N, gridDim.x * kWaves, blockIdx.x * kWaves + threadIdx.x / kWave, r0, r1);
  XVec xv = {xs, xs + C, xs + 2 * C};
  gemv_rows<R, U8>(a.hw, xv, r0, r1, lane, [&](int n, float sum) { a.logits[n] = (float)(h1)sum; });
}

// plain matmul, vector x matrix   (kernels/cuda/matmul.cpp:105-109)
struct Gemv {
  const h1* x;
  WMat w;
  void* y;
  int out_f32;
};

template <int R, bool U8>
__global__ __launch_bounds__(kThreads) void gemv_kernel(Gemv a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int K = a.w.K;
  h1* xs = reinterpret_cast<h1*>(smem);
  stage_vec<U8>(xs, a.x, K);
  if constexpr (U8) {
    stage_vec<true>(xs + K, a.w.ry, K);
    stage_vec<true>(xs + 2 * K, a.w.my, K);
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  int r0, r1;
  split_even(a.w.N, gridDim.x * kWaves, blockIdx.x * kWaves + threadIdx.x / kWave, r0, r1);
  XVec xv = {xs, xs + K, xs + 2 * K};
  gemv_rows<R, U8>(a.w, xv, r0, r1, lane, [&](int n, float sum) {
    if (a.out_f32)
      static_cast<float*>(a.y)[n] = sum;
    else
      static_cast<h1*>(a.y)[n] = (h1)sum;
  });
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static int check_weight(const frhip_weight* w, int K, int N) {
  if (!w || !w->data) return set_error(FRHIP_EINVAL, "weight is null");
  if (w->dtype != FRHIP_F16 && w->dtype != FRHIP_U8) return set_error(FRHIP_EINVAL, "weight dtype must be F16 or U8");
  if (K > 0 && w->K != K) return set_error(FRHIP_ESHAPE, "weight K does not match the activation length");
  if (N > 0 && w->N != N) return set_error(FRHIP_ESHAPE, "weight N does not match the output length");
  if (w->K <= 0 || w->N <= 0) return set_error(FRHIP_ESHAPE, "weight has an empty dimension");
  if (w->K % 16 != 0) return set_error(FRHIP_ESHAPE, "K must be a multiple of 16");
  if (reinterpret_cast<uintptr_t>(w->data) % 16 != 0) return set_error(FRHIP_EINVAL, "weight data must be 16-byte aligned");
  if (w->dtype == FRHIP_U8) {
    if (!w->mx || !w->rx || !w->my || !w->ry) return set_error(FRHIP_EINVAL, "uint8 weight without mx/rx/my/ry");
    if (reinterpret_cast<uintptr_t>(w->my) % 16 != 0 || reinterpret_cast<uintptr_t>(w->ry) % 16 != 0)
      return set_error(FRHIP_EINVAL, "my/ry must be 16-byte aligned");
  }
  return 0;
}

static int check_vec(const void* p, const char* what) {
  if (!p) return set_error(FRHIP_EINVAL, what);
  if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return set_error(FRHIP_EINVAL, what);
  return 0;
}

#define FR_TRY(expr)            \
  do {                          \
    int _e = (expr);            \
    if (_e != 0) return _e;     \
  } while (0)

static int check_embd(int C) {
  if (C <= 0 || C % 16 != 0 || C > 8 * kThreads) return set_error(FRHIP_ESHAPE, "n_embd must be a multiple of 16 and at most 4096");
  return 0;
}

// Rows in flight per wave: all of a wave's rows when that is few, else 4.
static int pick_r(long rows, int grid, bool u8) {
  long waves = (long)grid * kWaves;
  long per = (rows + waves - 1) / waves;
  int cap = u8 ? 4 : 6;
  if (per <= cap) return (int)(per < 1 ? 1 : per);
  return 4;
}

#define DISPATCH_R_U8(KERNEL, R, U8, GRID, LDS, STREAM, ARGS)                                          \
  do {                                                                                                 \
    if (U8) {                                                                                          \
      switch (R) {                                                                                     \
        case 1: hipLaunchKernelGGL((KERNEL<1, true>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 2: hipLaunchKernelGGL((KERNEL<2, true>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 3: hipLaunchKernelGGL((KERNEL<3, true>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        default: hipLaunchKernelGGL((KERNEL<4, true>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
      }                                                                                                \
    } else {                                                                                           \
      switch (R) {                                                                                     \
        case 1: hipLaunchKernelGGL((KERNEL<1, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 2: hipLaunchKernelGGL((KERNEL<2, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 3: hipLaunchKernelGGL((KERNEL<3, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 5: hipLaunchKernelGGL((KERNEL<5, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        case 6: hipLaunchKernelGGL((KERNEL<6, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
        default: hipLaunchKernelGGL((KERNEL<4, false>), dim3(GRID), dim3(kThreads), LDS, STREAM, ARGS); break; \
      }                                                                                                \
    }                                                                                                  \
  } while (0)

static int check_lds(size_t bytes) {
  if (bytes > 64 * 1024) return set_error(FRHIP_ESHAPE, "vector operands exceed 64 KB of LDS");
  return 0;
}

}  // namespace frhip

using namespace frhip;

extern "C" size_t frhip_decode_workspace_bytes(int C, int F) {
  // rwkv [C] | r [C] | vx [F] | x_mid [C]   (binary16), each 256-byte aligned
  auto al = [](size_t n) { return (n + 255) / 256 * 256; };
  if (C <= 0 || F <= 0) return 0;
  return al(2 * (size_t)C) * 3 + al(2 * (size_t)F);
}

namespace {
struct Workspace {
  h1 *rwkv, *r, *vx, *xmid;
};
Workspace carve(void* ws, int C, int F) {
  auto al = [](size_t n) { return (n + 255) / 256 * 256; };
  unsigned char* p = static_cast<unsigned char*>(ws);
  Workspace w;
  w.rwkv = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.r = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.xmid = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.vx = reinterpret_cast<h1*>(p);
  (void)F;
  return w;
}
}  // namespace

extern "C" int frhip_att_one_v4(int C, const void* x, const void* sx, const float* aa, const float* bb,
                                const float* pp, const void* ln_w, const void* ln_b, const void* k_mix,
                                const void* v_mix, const void* r_mix, const float* t_decay, const float* t_first,
                                const frhip_weight* kw, const frhip_weight* vw, const frhip_weight* rw,
                                const frhip_weight* ow, void* x_out, void* xx_out, float* aa_out, float* bb_out,
                                float* pp_out, void* workspace, frhip_stream s) {
  FR_TRY(check_embd(C));
  FR_TRY(check_vec(x, "x is null or misaligned"));
  FR_TRY(check_vec(sx, "sx is null or misaligned"));
  FR_TRY(check_vec(ln_w, "ln_w is null or misaligned"));
  FR_TRY(check_vec(ln_b, "ln_b is null or misaligned"));
  FR_TRY(check_vec(k_mix, "k_mix is null or misaligned"));
  FR_TRY(check_vec(v_mix, "v_mix is null or misaligned"));
  FR_TRY(check_vec(r_mix, "r_mix is null or misaligned"));
  FR_TRY(check_vec(x_out, "x_out is null or misaligned"));
  FR_TRY(check_vec(xx_out, "xx_out is null or misaligned"));
  FR_TRY(check_vec(workspace, "workspace is null or misaligned"));
  if (!aa || !bb || !pp || !t_decay || !t_first || !aa_out || !bb_out || !pp_out)
    return set_error(FRHIP_EINVAL, "att: null state or time parameter");
  if (xx_out == sx) return set_error(FRHIP_EINVAL, "att: xx_out must not alias sx");
  FR_TRY(check_weight(kw, C, C));
  FR_TRY(check_weight(vw, C, C));
  FR_TRY(check_weight(rw, C, C));
  FR_TRY(check_weight(ow, C, C));
  if (kw->dtype != vw->dtype || kw->dtype != rw->dtype) return set_error(FRHIP_EINVAL, "att: key/value/receptance dtypes differ");
  hipStream_t st = static_cast<hipStream_t>(s);
  Workspace w = carve(workspace, C, 16);
  const int grid = decode_grid();

  AttFrontV4 a;
  a.C = C;
  a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  a.mk = (const h1*)k_mix; a.mv = (const h1*)v_mix; a.mr = (const h1*)r_mix;
  a.aa = aa; a.bb = bb; a.pp = pp; a.td = t_decay; a.tf = t_first;
  a.kw = to_wmat(kw); a.vw = to_wmat(vw); a.rw = to_wmat(rw);
  a.xx_out = (h1*)xx_out; a.rwkv_out = w.rwkv;
  a.aa_out = aa_out; a.bb_out = bb_out; a.pp_out = pp_out;
  const bool u8 = kw->dtype == FRHIP_U8;
  size_t lds = 2 * (size_t)C * (u8 ? 9 : 3);
  FR_TRY(check_lds(lds));
  if (u8)
    hipLaunchKernelGGL(att_front_v4_kernel<true>, dim3(grid), dim3(kThreads), lds, st, a);
  else
    hipLaunchKernelGGL(att_front_v4_kernel<false>, dim3(grid), dim3(kThreads), lds, st, a);
  FR_TRY(check_launch("att_front_v4"));

  AttOutV4 b;
  b.C = C; b.rwkv = w.rwkv; b.x = (const h1*)x; b.ow = to_wmat(ow); b.x_out = (h1*)x_out;
  const bool ou8 = ow->dtype == FRHIP_U8;
  lds = 2 * (size_t)C * (ou8 ? 3 : 1);
  const int R = pick_r(C, grid, ou8);
  DISPATCH_R_U8(att_out_kernel, R, ou8, grid, lds, st, b);
  return check_launch("att_out");
}

extern "C" int frhip_ffn_one(int C, int F, const void* x, const void* sx, const void* ln_w, const void* ln_b,
                             const void* k_mix, const void* r_mix, const frhip_weight* kw, const frhip_weight* vw,
                             const frhip_weight* rw, void* x_out, void* xx_out, int post_div2, void* workspace,
                             frhip_stream s) {
  FR_TRY(check_embd(C));
  if (F <= 0 || F % 16 != 0) return set_error(FRHIP_ESHAPE, "n_ffn must be a positive multiple of 16");
  FR_TRY(check_vec(x, "x is null or misaligned"));
  FR_TRY(check_vec(sx, "sx is null or misaligned"));
  FR_TRY(check_vec(ln_w, "ln_w is null or misaligned"));
  FR_TRY(check_vec(ln_b, "ln_b is null or misaligned"));
  FR_TRY(check_vec(k_mix, "k_mix is null or misaligned"));
  FR_TRY(check_vec(r_mix, "r_mix is null or misaligned"));
  FR_TRY(check_vec(x_out, "x_out is null or misaligned"));
  FR_TRY(check_vec(xx_out, "xx_out is null or misaligned"));
  FR_TRY(check_vec(workspace, "workspace is null or misaligned"));
  if (xx_out == sx) return set_error(FRHIP_EINVAL, "ffn: xx_out must not alias sx");
  FR_TRY(check_weight(kw, C, F));
  FR_TRY(check_weight(vw, F, C));
  FR_TRY(check_weight(rw, C, C));
  if (kw->dtype != rw->dtype) return set_error(FRHIP_EINVAL, "ffn: key/receptance dtypes differ");
  hipStream_t st = static_cast<hipStream_t>(s);
  Workspace w = carve(workspace, C, F);
  const int grid = decode_grid();

  FfnFront a;
  a.C = C; a.F = F;
  a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  a.mk = (const h1*)k_mix; a.mr = (const h1*)r_mix;
  a.kw = to_wmat(kw); a.rw = to_wmat(rw);
  a.xx_out = (h1*)xx_out; a.r_out = w.r; a.vx_out = w.vx;
  const bool u8 = kw->dtype == FRHIP_U8;
  size_t lds = 2 * (size_t)C * (u8 ? 6 : 2);
  FR_TRY(check_lds(lds));
  int R = pick_r((long)C + F, grid, u8);
  DISPATCH_R_U8(ffn_front_kernel, R, u8, grid, lds, st, a);
  FR_TRY(check_launch("ffn_front"));

  FfnOut b;
  b.C = C; b.F = F; b.vx = w.vx; b.r = w.r; b.x = (const h1*)x; b.vw = to_wmat(vw);
  b.x_out = (h1*)x_out; b.div2 = post_div2 ? 1 : 0;
  const bool vu8 = vw->dtype == FRHIP_U8;
  lds = 2 * (size_t)F * (vu8 ? 3 : 1);
  FR_TRY(check_lds(lds));
  R = pick_r(C, grid, vu8);
  DISPATCH_R_U8(ffn_out_kernel, R, vu8, grid, lds, st, b);
  return check_launch("ffn_out");
}

extern "C" int frhip_head(int C, const void* x, const void* ln_w, const void* ln_b, const frhip_weight* head,
                          float* logits, frhip_stream s) {
  FR_TRY(check_embd(C));
  FR_TRY(check_vec(x, "x is null or misaligned"));
  FR_TRY(check_vec(ln_w, "ln_w is null or misaligned"));
  FR_TRY(check_vec(ln_b, "ln_b is null or misaligned"));
  if (!logits) return set_error(FRHIP_EINVAL, "logits is null");
  FR_TRY(check_weight(head, C, 0));
  Head a;
  a.C = C; a.x = (const h1*)x; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  a.hw = to_wmat(head); a.logits = logits;
  const bool u8 = head->dtype == FRHIP_U8;
  const int grid = decode_grid();
  size_t lds = 2 * (size_t)C * (u8 ? 3 : 1);
  FR_TRY(check_lds(lds));
  const int R = pick_r(head->N, grid, u8);
  DISPATCH_R_U8(head_kernel, R, u8, grid, lds, static_cast<hipStream_t>(s), a);
  return check_launch("head");
}

extern "C" int frhip_gemv(const void* x, const frhip_weight* w, void* y, int out_dtype, frhip_stream s) {
  FR_TRY(check_vec(x, "x is null or misaligned"));
  if (!y) return set_error(FRHIP_EINVAL, "y is null");
  if (out_dtype != FRHIP_F16 && out_dtype != FRHIP_F32) return set_error(FRHIP_EINVAL, "gemv: out_dtype must be F16 or F32");
  FR_TRY(check_weight(w, 0, 0));
  Gemv a;
  a.x = (const h1*)x; a.w = to_wmat(w); a.y = y; a.out_f32 = out_dtype == FRHIP_F32;
  const bool u8 = w->dtype == FRHIP_U8;
  const int grid = decode_grid();
  size_t lds = 2 * (size_t)w->K * (u8 ? 3 : 1);
  FR_TRY(check_lds(lds));
  const int R = pick_r(w->N, grid, u8);
  DISPATCH_R_U8(gemv_kernel, R, u8, grid, lds, static_cast<hipStream_t>(s), a);
  return check_launch("gemv");
}
