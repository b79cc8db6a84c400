// Device-side helpers shared by the gfx950 kernels: binary16 vector types, DPP
// wavefront reductions, the fused uint8 dequantisation, and row-times-vector dot
// products over output-major weights.
//
// Rounding discipline: the reference's fp16 path rounds to half after every
// elementwise operation (kernels/cuda/att.cu:90-175, ffn.cu:15-60).  All _Float16
// expressions below are therefore evaluated with contraction OFF; fused
// multiply-adds appear only where the reference has one (__hfma) or where the
// dequantisation formula specifies one.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#pragma clang fp contract(off)

namespace frhip {

typedef _Float16 h1;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// ---- cross-lane reductions (DPP, no LDS traffic) ---------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes; every lane receives the same value.  The association
// order is fixed, so results are reproducible run to run.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_mov<0x141>(v);  // row_half_mirror
  v += dpp_mov<0x140>(v);  // row_mirror      -> each 16-lane row holds its sum
  float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return ((a + b) + c) + d;
}

// Sum over a workgroup of NWAVES wavefronts; `red` is NWAVES floats of LDS.
// All threads must call it; it contains two barriers.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  __syncthreads();  // protect `red` from a previous use
  if ((threadIdx.x & (kWave - 1)) == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; i++) t += red[i];
  return t;
}

// ---- elementwise pieces, rounding as the reference does ---------------------
// kernels/cuda/att.cu:106-107: h(h(xx*m) + h(sx*h(1-m)))
__device__ __forceinline__ h1 mix1(h1 xx, h1 sx, h1 m) { return (xx * m) + (sx * ((h1)1.0f - m)); }

// kernels/cuda/att.cu:154-159: evaluated in double, narrowed to float, then to half
__device__ __forceinline__ h1 sigmoid_h(h1 x) {
  double s = 1.0 / (1.0 + exp(-(double)(float)x));
  return (h1)(float)s;
}

// kernels/cuda/att.cu:145-152
__device__ __forceinline__ h1 silu_h(h1 x) {
  h1 e = (h1)expf(-(float)x);
  return (h1)((float)x / (float)((h1)1.0f + e));  // correctly rounded fp32 quotient == rounded half quotient
}

// ---- uint8 dequantisation ----------------------------------------------------
// All binary16, round-to-nearest-even:
//   c255 = rx[n] / 255 ; a = c255 * ry[k] ; b = mx[n] + my[k] ; w^ = fma(q, a, b)
__device__ __forceinline__ h1 dequant_c255(h1 rx) { return (h1)((float)rx / 255.0f); }

// Two codes at once.  `word` holds 4 codes; HI selects bytes 2,3 instead of 0,1.
// v_perm_b32 plants each code in the mantissa of 1024.0 (0x6400 | q == 1024 + q,
// exact), the subtraction of 1024 is exact, the rest is the formula above.
template <int HI>
__device__ __forceinline__ h2 dequant_pair(uint32_t word, h2 c255, h2 mx, h2 ry, h2 my) {
  const uint32_t sel = HI ? 0x04030402u : 0x04010400u;
  uint32_t planted = __builtin_amdgcn_perm(0x64646464u, word, sel);
  h2 q = __builtin_bit_cast(h2, planted) - (h2){(h1)1024.0f, (h1)1024.0f};
  h2 a = c255 * ry;
  h2 b = mx + my;
  return __builtin_elementwise_fma(q, a, b);
}

__device__ __forceinline__ float dot2acc(h2 a, h2 b, float acc) {
  return __builtin_amdgcn_fdot2(a, b, acc, false);
}

__device__ __forceinline__ float dot8acc(h8 w, h8 x, float acc) {
  acc = dot2acc(w.s01, x.s01, acc);
  acc = dot2acc(w.s23, x.s23, acc);
  acc = dot2acc(w.s45, x.s45, acc);
  acc = dot2acc(w.s67, x.s67, acc);
  return acc;
}

// A vector operand staged in LDS for one matrix: the activation and, for uint8
// weights, the per-row (k-indexed) offset and range.
struct XVec {
  const h1* x;
  const h1* ry;
  const h1* my;
};

// Per-row (n-indexed) constants of a uint8 row.
struct RowQ {
  h1 c255;
  h1 mx;
};

// Position, in units of 8 halves, at which group g of a K-element vector is staged.
// binary16 weights: in order.  uint8 weights: split layout (see dot_rows).
template <bool U8>
__device__ __forceinline__ int stage_pos(int g, int K) {
  if constexpr (U8) return (g & 1) * (K >> 4) + (g >> 1);
  return g;
}

// Copy a K-element binary16 vector from global memory into LDS in staged order.
template <bool U8>
__device__ __forceinline__ void stage_vec(h1* dst, const h1* src, int K) {
  for (int g = threadIdx.x; g < (K >> 3); g += blockDim.x)
    reinterpret_cast<h8*>(dst)[stage_pos<U8>(g, K)] = reinterpret_cast<const h8*>(src)[g];
}

// Per-lane partial dot products of R weight rows with LDS-resident vectors.
// rows[r] points at K contiguous elements (binary16, or uint8 codes when U8).
// K must be a multiple of 8 (binary16) or 16 (uint8).  Weight rows are streamed
// once, so they are loaded non-temporally.
template <int R, bool U8>
__device__ __forceinline__ void dot_rows(const void* const (&rows)[R], const XVec (&xv)[R],
                                         const RowQ (&rq)[R], int K, int lane, float (&acc)[R]) {
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;
  if constexpr (!U8) {
    const int nchunk = K >> 3;
#pragma unroll 2
    for (int c = lane; c < nchunk; c += kWave) {
      h8 w[R];
#pragma unroll
      for (int r = 0; r < R; r++) w[r] = __builtin_nontemporal_load(reinterpret_cast<const h8*>(rows[r]) + c);
#pragma unroll
      for (int r = 0; r < R; r++) {
        h8 x = reinterpret_cast<const h8*>(xv[r].x)[c];
        acc[r] = dot8acc(w[r], x, acc[r]);
      }
    }
  } else {
    const int nchunk = K >> 4;
#pragma unroll 2
    for (int c = lane; c < nchunk; c += kWave) {
      u32x4 w[R];
#pragma unroll
      for (int r = 0; r < R; r++) w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(rows[r]) + c);
#pragma unroll
      for (int r = 0; r < R; r++) {
        // uint8 operands are staged "split": 8-element groups with even index in the
        // first half of the array, odd ones in the second, so that consecutive lanes
        // read consecutive 16-byte words of LDS (no bank conflicts).
        const h8* xp = reinterpret_cast<const h8*>(xv[r].x) + c;
        const h8* ryp = reinterpret_cast<const h8*>(xv[r].ry) + c;
        const h8* myp = reinterpret_cast<const h8*>(xv[r].my) + c;
        const h2 c2 = {rq[r].c255, rq[r].c255};
        const h2 m2 = {rq[r].mx, rq[r].mx};
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
          h8 x = xp[hh * nchunk], ry = ryp[hh * nchunk], my = myp[hh * nchunk];
          uint32_t w0 = w[r][2 * hh], w1 = w[r][2 * hh + 1];
          acc[r] = dot2acc(dequant_pair<0>(w0, c2, m2, ry.s01, my.s01), x.s01, acc[r]);
          acc[r] = dot2acc(dequant_pair<1>(w0, c2, m2, ry.s23, my.s23), x.s23, acc[r]);
          acc[r] = dot2acc(dequant_pair<0>(w1, c2, m2, ry.s45, my.s45), x.s45, acc[r]);
          acc[r] = dot2acc(dequant_pair<1>(w1, c2, m2, ry.s67, my.s67), x.s67, acc[r]);
        }
      }
    }
  }
}

}  // namespace frhip
