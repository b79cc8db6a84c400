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
typedef float f32x4 __attribute__((ext_vector_type(4)));

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

// As block_sum with a single barrier: `red` must not have been written since the
// workgroup's previous barrier-separated use of it (callers alternate between two arrays).
template <int NWAVES>
__device__ __forceinline__ float block_sum1(float v, float* red) {
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; i++) t += red[i];
  return t;
}

// ---- elementwise pieces, rounding as the reference does ---------------------
// kernels/cuda/att.cu:106-107: h(h(xx*m) + h(sx*h(1-m)))
__device__ __forceinline__ h1 mix1(h1 xx, h1 sx, h1 m) { return (xx * m) + (sx * ((h1)1.0f - m)); }

// kernels/cuda/att.cu:154-159: evaluated in double, narrowed to float, then to half.
// The double evaluation costs hundreds of cycles at the tail of a wave, so the value is first
// formed in fp32 (a few units in the last place of error); only when that lies so close to the
// midpoint of two binary16 values that the error could change the rounding, or in the binary16
// subnormal range, is the double path taken.  The result is the double path's bit for bit.
__device__ __forceinline__ h1 sigmoid_h_exact(h1 x) {
  const double s = 1.0 / (1.0 + exp(-(double)(float)x));
  return (h1)(float)s;
}
// The fp32 value rounded to binary16; *safe says whether that is certainly sigmoid_h_exact's result.
__device__ __forceinline__ h1 sigmoid_h_fast(h1 x, bool* safe) {
  const float xf = (float)x;
  const float s32 = 1.0f / (1.0f + expf(-xf));
  const uint32_t frac = __float_as_uint(s32) & 0x1FFFu;  // the 13 fp32 mantissa bits binary16 drops
  *safe = s32 > 1e-4f && (frac < 0x1000u - 64u || frac > 0x1000u + 64u);
  return (h1)s32;
}
__device__ __forceinline__ h1 sigmoid_h(h1 x) {
  bool safe;
  const h1 y = sigmoid_h_fast(x, &safe);
  return safe ? y : sigmoid_h_exact(x);
}

// kernels/cuda/att.cu:145-152
__device__ __forceinline__ h1 silu_h(h1 x) {
  h1 e = (h1)expf(-(float)x);
  return (h1)((float)x / (float)((h1)1.0f + e));  // correctly rounded fp32 quotient == rounded half quotient
}

// ---- uint8 dequantisation ----------------------------------------------------
// Evaluated in fp32 with one final round-to-nearest-even to binary16:
//   c = rx[n] / 255 ; a = c * ry[k] ; b = mx[n] + my[k] ; w^ = h(fma(q, a, b))
// (every fp32 operation correctly rounded, no contraction besides the stated fma).
__device__ __forceinline__ float dequant_c(h1 rx) { return (float)rx / 255.0f; }

// Two codes at once.  `word` holds 4 codes; HI selects bytes 2,3 instead of 0,1.
template <int HI>
__device__ __forceinline__ h2 dequant_pair(uint32_t word, float c, float mx, h2 ry, h2 my) {
  const float q0 = (float)((word >> (HI ? 16 : 0)) & 0xffu);
  const float q1 = (float)((word >> (HI ? 24 : 8)) & 0xffu);
  const float a0 = c * (float)ry.x, a1 = c * (float)ry.y;
  const float b0 = mx + (float)my.x, b1 = mx + (float)my.y;
  return (h2){(h1)__builtin_fmaf(q0, a0, b0), (h1)__builtin_fmaf(q1, a1, b1)};
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

// Position, in units of 8 halves, at which group g of a K-element vector is staged.
// binary16 weights: in order.  uint8 weights: split layout (8-element groups with even index
// in the first half, odd ones in the second, so that consecutive lanes read consecutive
// 16-byte LDS words when a lane's 16 codes span two groups).
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

}  // namespace frhip
