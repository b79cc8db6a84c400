// Primitive operators of the `hip` device: the ones kernels/kernels.h names that are
// not fused into the one-token kernels (layernorm, groupnorm, cast_dtype, fill_,
// scalar_div_, vgather), weight preparation, and the greedy sampler's argmax.
#include "device_utils.h"
#include "frhip_internal.h"
#include "gemm.h"

#pragma clang fp contract(off)

namespace frhip {

// ---- layernorm over rows: one workgroup (256 threads) per row ----------------
// kernels/cuda/layer_norm.cu:101-130.  fp32 statistics (two passes over registers
// or, for long rows, over memory), eps 1e-5.  binary16: the normalised value is
// rounded to half before the affine, which is done in half (layer_norm.cu:60-69).
template <typename T>
__global__ __launch_bounds__(256) void layernorm_rows_kernel(const T* __restrict__ x, const T* __restrict__ gamma,
                                                             const T* __restrict__ beta, T* __restrict__ y, int cols) {
  __shared__ float red[4];
  const T* xr = x + (size_t)blockIdx.x * cols;
  T* yr = y + (size_t)blockIdx.x * cols;
  float s = 0.f;
  for (int i = threadIdx.x; i < cols; i += 256) s += (float)xr[i];
  const float mean = block_sum<4>(s, red) / (float)cols;
  float q = 0.f;
  for (int i = threadIdx.x; i < cols; i += 256) {
    float d = (float)xr[i] - mean;
    q += d * d;
  }
  float var = block_sum<4>(q, red) / (float)cols;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
  for (int i = threadIdx.x; i < cols; i += 256) {
    float n = ((float)xr[i] - mean) * inv;
    if constexpr (sizeof(T) == 2) {
      yr[i] = ((T)n * gamma[i]) + beta[i];
    } else {
      yr[i] = n * gamma[i] + beta[i];
    }
  }
}

// ---- groupnorm, fp32: one wavefront per (row, group) -------------------------
// kernels/cuda/group_norm.cu:322-357 (instances = rows*groups, eps 1e-5).
__global__ __launch_bounds__(256) void groupnorm_f32_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                            const float* __restrict__ beta, float* __restrict__ y,
                                                            int instances, int groups, int gs) {
  const int inst = blockIdx.x * 4 + threadIdx.x / kWave;
  if (inst >= instances) return;  // whole wave exits together
  const int lane = threadIdx.x & (kWave - 1);
  const int g = inst % groups;
  const float* xr = x + (size_t)inst * gs;
  float* yr = y + (size_t)inst * gs;
  float s = 0.f;
  for (int i = lane; i < gs; i += kWave) s += xr[i];
  const float mean = wave_sum(s) / (float)gs;
  float q = 0.f;
  for (int i = lane; i < gs; i += kWave) {
    float d = xr[i] - mean;
    q += d * d;
  }
  float var = wave_sum(q) / (float)gs;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
  for (int i = lane; i < gs; i += kWave) yr[i] = (xr[i] - mean) * inv * gamma[g * gs + i] + beta[g * gs + i];
}

template <typename S, typename D>
__global__ void cast_kernel(const S* __restrict__ src, D* __restrict__ dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = (D)src[i];
}

template <typename T>
__global__ void fill_kernel(T* x, T v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = v;
}

// kernels/cuda/element_wise.cu:8-12: x = x / half(val)
__global__ void scalar_div_f16_kernel(h1* x, h1 d, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = (h1)((float)x[i] / (float)d);  // rounded fp32 quotient == rounded half quotient
}

__global__ void gather_rows_kernel(const unsigned char* __restrict__ table, const int32_t* __restrict__ ids,
                                   unsigned char* __restrict__ out, int row_bytes) {
  const u32x4* src = reinterpret_cast<const u32x4*>(table + (size_t)ids[blockIdx.x] * row_bytes);
  u32x4* dst = reinterpret_cast<u32x4*>(out + (size_t)blockIdx.x * row_bytes);
  for (int i = threadIdx.x; i < row_bytes / 16; i += blockDim.x) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void embed_ring_kernel(const unsigned char* __restrict__ table, int n_rows,
                                                         int row_bytes, const int32_t* ring, int ring_len,
                                                         uint32_t* counter, unsigned char* __restrict__ out) {
  __shared__ int row;
  if (threadIdx.x == 0) {
    const uint32_t c = *counter;
    int id = ring[c % (uint32_t)ring_len];
    id = id < 0 ? 0 : (id >= n_rows ? n_rows - 1 : id);
    row = id;
    *counter = c + 1;
  }
  __syncthreads();
  const u32x4* src = reinterpret_cast<const u32x4*>(table + (size_t)row * row_bytes);
  u32x4* dst = reinterpret_cast<u32x4*>(out);
  for (int i = threadIdx.x; i < row_bytes / 16; i += blockDim.x) dst[i] = src[i];
}

// Token feed of a greedy loop that stays on the device: the token of this step is the arg-max of the
// previous step's logits, taken from that step's per-slice {value, index} pairs (greater value, then
// smaller index; index n_rows or beyond, i.e. no finite maximum, gives token 0: the host's rule).
// The token goes to ids[*counter % ids_len] for the host to read later, *counter advances, and the
// token's row of `table` is copied to `out`.
__global__ __launch_bounds__(256) void embed_argmax_kernel(const unsigned char* __restrict__ table, int n_rows,
                                                           int row_bytes, const float* pairs, int npairs, int32_t* ids,
                                                           int ids_len, uint32_t* counter, unsigned char* __restrict__ out) {
  __shared__ int row;
  if (threadIdx.x < 64) {
    float best = -INFINITY;
    int idx = n_rows;
    for (int b = threadIdx.x; b < npairs; b += 64) {
      const float v = pairs[2 * b];
      const int i = reinterpret_cast<const int32_t*>(pairs)[2 * b + 1];
      if (v > best || (v == best && i < idx)) {
        best = v;
        idx = i;
      }
    }
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off);
      const int oi = __shfl_xor(idx, off);
      if (ov > best || (ov == best && oi < idx)) {
        best = ov;
        idx = oi;
      }
    }
    if (threadIdx.x == 0) {
      const int id = (idx >= 0 && idx < n_rows) ? idx : 0;
      const uint32_t c = *counter;
      ids[c % (uint32_t)ids_len] = id;
      *counter = c + 1;
      row = id;
    }
  }
  __syncthreads();
  const u32x4* src = reinterpret_cast<const u32x4*>(table + (size_t)row * row_bytes);
  u32x4* dst = reinterpret_cast<u32x4*>(out);
  for (int i = threadIdx.x; i < row_bytes / 16; i += blockDim.x) dst[i] = src[i];
}

// [K][N] -> [N][K] through a 64x64 LDS tile (+1 padding against bank conflicts).
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ src, T* __restrict__ dst, int K, int N) {
  __shared__ T tile[64][65];
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    int k = k0 + r, n = n0 + tx;
    if (k < K && n < N) tile[r][tx] = src[(size_t)k * N + n];
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    int n = n0 + r, k = k0 + tx;
    if (k < K && n < N) dst[(size_t)n * K + k] = tile[tx][r];
  }
}

// Packed uint8 [N][K] -> packed binary16 [N][K]; thread handles 4 codes of one row.
__global__ void dequant_u8_kernel(const uint32_t* __restrict__ q, const h1* __restrict__ mx, const h1* __restrict__ rx,
                                  const h1* __restrict__ my, const h1* __restrict__ ry, h4* __restrict__ out, int K,
                                  int N) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // index of a 4-code word
  const size_t words = (size_t)N * (K >> 2);
  if (i >= words) return;
  const int n = (int)(i / (K >> 2));
  const int k = (int)(i % (K >> 2)) * 4;
  const float c2 = dequant_c(rx[n]);
  const float m2 = (float)mx[n];
  const uint32_t w = q[i];
  h2 ry01 = {ry[k], ry[k + 1]}, ry23 = {ry[k + 2], ry[k + 3]};
  h2 my01 = {my[k], my[k + 1]}, my23 = {my[k + 2], my[k + 3]};
  h2 lo = dequant_pair<0>(w, c2, m2, ry01, my01);
  h2 hi = dequant_pair<1>(w, c2, m2, ry23, my23);
  out[i] = (h4){lo.x, lo.y, hi.x, hi.y};
}

// The same, 16 codes per thread (K a multiple of 16): one 16-byte load of codes, two each of ry
// and my, two 16-byte stores.  The seq-mode products expand a launch's uint8 weights with this
// before the binary16 GEMM, so it runs at copy rate or the expansion eats what it saves: with
// 4 codes per thread (a 64-bit division, eight 2-byte loads of ry/my per word) the 2560 x 2560
// matrices of a 3B model took 8.0 us each, 2.4 TB/s of traffic.
__device__ __forceinline__ void dequant_chunk16(const u32x4* __restrict__ q, const h1* __restrict__ mx, const h1* __restrict__ rx,
                                                const h1* __restrict__ my, const h1* __restrict__ ry, h8* __restrict__ out,
                                                int K16, unsigned i) {
  const unsigned n = i / (unsigned)K16;
  const int k = (int)(i - n * (unsigned)K16) * 16;
  const float c2 = dequant_c(rx[n]);
  const float m2 = (float)mx[n];
  const u32x4 w = __builtin_nontemporal_load(q + i);
#pragma unroll
  for (int hh = 0; hh < 2; hh++) {
    const h8 ryv = *reinterpret_cast<const h8*>(ry + k + hh * 8);
    const h8 myv = *reinterpret_cast<const h8*>(my + k + hh * 8);
    const uint32_t w0 = w[2 * hh], w1 = w[2 * hh + 1];
    const h2 p0 = dequant_pair<0>(w0, c2, m2, ryv.s01, myv.s01);
    const h2 p1 = dequant_pair<1>(w0, c2, m2, ryv.s23, myv.s23);
    const h2 p2 = dequant_pair<0>(w1, c2, m2, ryv.s45, myv.s45);
    const h2 p3 = dequant_pair<1>(w1, c2, m2, ryv.s67, myv.s67);
    out[(size_t)i * 2 + hh] = (h8){p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
  }
}

__global__ __launch_bounds__(256) void dequant_u8x16_kernel(const u32x4* __restrict__ q, const h1* __restrict__ mx,
                                                            const h1* __restrict__ rx, const h1* __restrict__ my,
                                                            const h1* __restrict__ ry, h8* __restrict__ out, int K16,
                                                            unsigned chunks) {
  const unsigned i = blockIdx.x * 256u + threadIdx.x;  // index of a 16-code chunk
  if (i < chunks) dequant_chunk16(q, mx, rx, my, ry, out, K16, i);
}

// Up to four matrices over the same K in one launch (blockIdx.y picks the matrix): the weights of
// a grouped product (k, v, r, g or ffn r, k) are expanded together instead of in four launches of
// a few microseconds each.
struct DequantGroup {
  const u32x4* q[4];
  const h1 *mx[4], *rx[4], *my[4], *ry[4];
  h8* out[4];
  unsigned chunks[4];
  int K16;
};
__global__ __launch_bounds__(256) void dequant_u8x16_group_kernel(DequantGroup g) {
  const int s = blockIdx.y;
  const unsigned i = blockIdx.x * 256u + threadIdx.x;
  if (i < g.chunks[s]) dequant_chunk16(g.q[s], g.mx[s], g.rx[s], g.my[s], g.ry[s], g.out[s], g.K16, i);
}

__global__ __launch_bounds__(256) void copy_probe_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

__global__ __launch_bounds__(512) void read_probe_kernel(const u32x4* __restrict__ src, size_t n, uint32_t* sink) {
  u32x4 acc = {0, 0, 0, 0};
  const size_t stride = (size_t)gridDim.x * 512;
  size_t i = (size_t)blockIdx.x * 512 + threadIdx.x;
  for (; i + 3 * stride < n; i += 4 * stride) {
    u32x4 a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride);
    u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride), d = __builtin_nontemporal_load(src + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  uint32_t v = acc.x ^ acc.y ^ acc.z ^ acc.w;
  for (int off = 32; off > 0; off >>= 1) v ^= __shfl_xor(v, off);
  if ((threadIdx.x & 63) == 0 && threadIdx.x == 0) sink[blockIdx.x] = v;
}

// The same over nblocks contiguous slices, one workgroup of 256 threads each: block b writes the
// largest value of slice b and its (global) index, first occurrence on ties, as the pair
// {float, int32} number b.  A slice is len elements (a multiple of 4; the last may be short or
// empty: it reports -inf at index n).  The caller reduces the pairs (greater value, then smaller
// index): with the logits in one slab that is 64 pairs instead of 65 536 values.
__global__ __launch_bounds__(256) void argmax_blocks_f32_kernel(const float* __restrict__ x, int n, int len,
                                                              float* pairs, float* mirror) {
  __shared__ float bv[4];
  __shared__ int bi[4];
  const int lo = blockIdx.x * len;
  const int hi = lo + len < n ? lo + len : n;
  float best = -INFINITY;
  int idx = n;
  // thread t scans groups of 4 at lo + 4t, lo + 4t + 1024, ...: increasing indices, so '>' keeps the first
  for (int i = lo + 4 * (int)threadIdx.x; i < hi; i += 1024) {
    if (i + 4 <= hi) {
      const float4 v = *reinterpret_cast<const float4*>(x + i);
      if (v.x > best) { best = v.x; idx = i; }
      if (v.y > best) { best = v.y; idx = i + 1; }
      if (v.z > best) { best = v.z; idx = i + 2; }
      if (v.w > best) { best = v.w; idx = i + 3; }
    } else {
      for (int j = i; j < hi; j++)
        if (x[j] > best) { best = x[j]; idx = j; }
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    float ov = __shfl_xor(best, off);
    int oi = __shfl_xor(idx, off);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    bv[threadIdx.x >> 6] = best;
    bi[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
        best = bv[w];
        idx = bi[w];
      }
    pairs[2 * blockIdx.x] = best;
    reinterpret_cast<int32_t*>(pairs)[2 * blockIdx.x + 1] = idx;
    if (mirror) {  // a second copy, e.g. in pinned host memory beside the logits
      mirror[2 * blockIdx.x] = best;
      reinterpret_cast<int32_t*>(mirror)[2 * blockIdx.x + 1] = idx;
    }
  }
}

// Index of the maximum, first occurrence on ties; single workgroup of 1024 threads.
__global__ __launch_bounds__(1024) void argmax_f32_kernel(const float* __restrict__ x, int n, int32_t* out) {
  __shared__ float bv[16];
  __shared__ int bi[16];
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < n; i += 1024) {
    float v = x[i];
    if (v > best || (v == best && i < idx)) {
      best = v;
      idx = i;
    }
  }
  for (int off = 32; off > 0; off >>= 1) {
    float ov = __shfl_xor(best, off);
    int oi = __shfl_xor(idx, off);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    bv[threadIdx.x >> 6] = best;
    bi[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; w++)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
        best = bv[w];
        idx = bi[w];
      }
    *out = idx == 0x7fffffff ? 0 : idx;
  }
}

int dequant_u8_async(const unsigned char* q, const h1* mx, const h1* rx, const h1* my, const h1* ry, h1* dst, int K, int N,
                     hipStream_t st) {
  const size_t chunks = (size_t)N * (K / 16);
  if (K % 16 == 0 && chunks < (1u << 31) && reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(ry) % 16 == 0 && reinterpret_cast<uintptr_t>(my) % 16 == 0) {
    hipLaunchKernelGGL(dequant_u8x16_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, (const u32x4*)q, mx, rx, my, ry,
                       (h8*)dst, K / 16, (unsigned)chunks);
    return check_launch("dequant_u8");
  }
  const size_t words = (size_t)N * (K / 4);
  hipLaunchKernelGGL(dequant_u8_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, st, (const uint32_t*)q, mx, rx, my, ry,
                     (h4*)dst, K, N);
  return check_launch("dequant_u8");
}

int dequant_u8_group_async(int nseg, const unsigned char* const* q, const h1* const* mx, const h1* const* rx, const h1* const* my,
                           const h1* const* ry, h1* const* dst, int K, const int* N, hipStream_t st) {
  bool fast = K % 16 == 0 && nseg >= 2 && nseg <= 4;
  unsigned most = 0;
  DequantGroup g;
  for (int s = 0; fast && s < nseg; s++) {
    const size_t chunks = (size_t)N[s] * (K / 16);
    fast = chunks < (1u << 31) && reinterpret_cast<uintptr_t>(q[s]) % 16 == 0 && reinterpret_cast<uintptr_t>(dst[s]) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(ry[s]) % 16 == 0 && reinterpret_cast<uintptr_t>(my[s]) % 16 == 0;
    g.q[s] = reinterpret_cast<const u32x4*>(q[s]);
    g.mx[s] = mx[s]; g.rx[s] = rx[s]; g.my[s] = my[s]; g.ry[s] = ry[s];
    g.out[s] = reinterpret_cast<h8*>(dst[s]);
    g.chunks[s] = (unsigned)chunks;
    most = g.chunks[s] > most ? g.chunks[s] : most;
  }
  if (!fast) {
    for (int s = 0; s < nseg; s++)
      if (int rc = dequant_u8_async(q[s], mx[s], rx[s], my[s], ry[s], dst[s], K, N[s], st)) return rc;
    return 0;
  }
  for (int s = nseg; s < 4; s++) {
    g.q[s] = g.q[0]; g.mx[s] = g.mx[0]; g.rx[s] = g.rx[0]; g.my[s] = g.my[0]; g.ry[s] = g.ry[0]; g.out[s] = g.out[0];
    g.chunks[s] = 0;
  }
  g.K16 = K / 16;
  hipLaunchKernelGGL(dequant_u8x16_group_kernel, dim3((most + 255) / 256, nseg), dim3(256), 0, st, g);
  return check_launch("dequant_u8 (group)");
}

// ---- matrix-core rate probe (diagnostic) -----------------------------------------------------
// Nothing but v_mfma_f32_32x32x16_f16 on register operands: six independent accumulators per wave
// so that the matrix pipe never waits for a result.  Each wave also reads the core clock counter
// and the constant 100 MHz counter around its loop, which gives the clock the compute unit ran at.
typedef float f32x16 __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(512) void mfma_probe_kernel(const h8* __restrict__ operands, int iters, float* __restrict__ sink,
                                                         unsigned long long* __restrict__ clocks) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  const h8 a = operands[2 * (gid & 4095)], b = operands[2 * (gid & 4095) + 1];
  f32x16 acc[6];
#pragma unroll
  for (int i = 0; i < 6; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) acc[i][j] = 0.f;
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < 6; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 6; i++)
#pragma unroll
    for (int j = 0; j < 16; j++) t += acc[i][j];
  sink[gid] = t;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    const int w = gid / kWave;
    clocks[2 * w] = c1 - c0;
    clocks[2 * w + 1] = w1 - w0;
  }
}

// ---- shape operators (kernels/cuda/slice.cu:17-36, cat.cu:28-52, transpose.cu:16-34) ----------
// Index math over at most four dimensions with the shapes passed by value: no device allocation
// and no blocking copy per call.
struct Dims4 {
  int n[4];
};

// dst[i0..i3] = src[start + i * interval] per dimension
template <typename T>
__global__ __launch_bounds__(256) void slice_kernel(const T* __restrict__ src, T* __restrict__ dst, Dims4 src_shape,
                                                    Dims4 dst_shape, Dims4 start, Dims4 interval, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  size_t rem = i, off = 0, stride = 1;
#pragma unroll
  for (int d = 3; d >= 0; d--) {
    const size_t idx = rem % (size_t)dst_shape.n[d];
    rem /= (size_t)dst_shape.n[d];
    off += ((size_t)start.n[d] + idx * (size_t)interval.n[d]) * stride;
    stride *= (size_t)src_shape.n[d];
  }
  dst[i] = src[off];
}

// out [left][a_mid + b_mid][right] from a [left][a_mid][right] and b [left][b_mid][right]
template <typename T>
__global__ __launch_bounds__(256) void cat_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
                                                  size_t a_mid, size_t b_mid, size_t right, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t r = i % right, m = (i / right) % (a_mid + b_mid), l = i / (right * (a_mid + b_mid));
  out[i] = m < a_mid ? a[(l * a_mid + m) * right + r] : b[(l * b_mid + (m - a_mid)) * right + r];
}

// dst = src with dimensions dim_a and dim_b exchanged
template <typename T>
__global__ __launch_bounds__(256) void transpose_nd_kernel(const T* __restrict__ src, T* __restrict__ dst, Dims4 src_shape,
                                                           int dim_a, int dim_b, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  Dims4 ds = src_shape;
  const int t = ds.n[dim_a];
  ds.n[dim_a] = ds.n[dim_b];
  ds.n[dim_b] = t;
  int idx[4];
  size_t rem = i;
#pragma unroll
  for (int d = 3; d >= 0; d--) {
    idx[d] = (int)(rem % (size_t)ds.n[d]);
    rem /= (size_t)ds.n[d];
  }
  const int u = idx[dim_a];
  idx[dim_a] = idx[dim_b];
  idx[dim_b] = u;
  size_t off = 0;
#pragma unroll
  for (int d = 0; d < 4; d++) off = off * (size_t)src_shape.n[d] + (size_t)idx[d];
  dst[i] = src[off];
}

// silu.  binary16 rounds as the fused attention path does (kernels/cuda/att.cu:145-152):
// x / (1 + half(exp(-x))) in half.  (The reference's standalone operator, activations/silu.cu:19,28,
// evaluates x / (1 - exp(x)), which is not SiLU; nothing on its CUDA path calls it.)
__global__ void silu_f16_kernel(const h1* __restrict__ x, h1* __restrict__ y, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = silu_h(x[i]);
}
__global__ void silu_f32_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = x[i] / (1.0f + expf(-x[i]));
}

}  // namespace frhip

using namespace frhip;

static unsigned blocks_for(size_t n, unsigned per) { return (unsigned)((n + per - 1) / per); }

namespace {
// Right-align `ndim` values into four slots, filling the leading ones with `fill`.
bool to_dims4(const int* v, int ndim, int fill, Dims4* out) {
  if (ndim < 1 || ndim > 4 || !v) return false;
  for (int d = 0; d < 4; d++) out->n[d] = fill;
  for (int d = 0; d < ndim; d++) out->n[4 - ndim + d] = v[d];
  return true;
}
template <typename F>
int by_elem_bytes(int elem_bytes, F&& f) {
  switch (elem_bytes) {
    case 1: f(uint8_t{}); return 0;
    case 2: f(uint16_t{}); return 0;
    case 4: f(uint32_t{}); return 0;
    default: return set_error(FRHIP_EINVAL, "shape operator: elem_bytes must be 1, 2 or 4");
  }
}
}  // namespace

extern "C" {

int frhip_layernorm(const void* x, const void* gamma, const void* beta, void* y, int rows, int cols, int dtype,
                    frhip_stream s) {
  if (!x || !gamma || !beta || !y) return set_error(FRHIP_EINVAL, "layernorm: null pointer");
  if (rows < 0 || cols <= 0) return set_error(FRHIP_ESHAPE, "layernorm: bad shape");
  if (rows == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  if (dtype == FRHIP_F16)
    hipLaunchKernelGGL(layernorm_rows_kernel<h1>, dim3(rows), dim3(256), 0, st, (const h1*)x, (const h1*)gamma,
                       (const h1*)beta, (h1*)y, cols);
  else if (dtype == FRHIP_F32)
    hipLaunchKernelGGL(layernorm_rows_kernel<float>, dim3(rows), dim3(256), 0, st, (const float*)x,
                       (const float*)gamma, (const float*)beta, (float*)y, cols);
  else
    return set_error(FRHIP_EINVAL, "layernorm: dtype must be F16 or F32");
  return check_launch("layernorm");
}

int frhip_groupnorm_f32(const float* x, int groups, const float* gamma, const float* beta, float* y, int rows,
                        int cols, frhip_stream s) {
  if (!x || !gamma || !beta || !y) return set_error(FRHIP_EINVAL, "groupnorm: null pointer");
  if (rows < 0 || cols <= 0 || groups <= 0 || cols % groups != 0) return set_error(FRHIP_ESHAPE, "groupnorm: bad shape");
  if (rows == 0) return 0;
  const int inst = rows * groups;
  hipLaunchKernelGGL(groupnorm_f32_kernel, dim3((inst + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(s), x, gamma,
                     beta, y, inst, groups, cols / groups);
  return check_launch("groupnorm");
}

int frhip_cast(const void* src, int sd, void* dst, int dd, size_t n, frhip_stream s) {
  if (!src || !dst) return set_error(FRHIP_EINVAL, "cast: null pointer");
  if (n == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  if (sd == FRHIP_F16 && dd == FRHIP_F32)
    hipLaunchKernelGGL((cast_kernel<h1, float>), dim3(blocks_for(n, 256)), dim3(256), 0, st, (const h1*)src, (float*)dst, n);
  else if (sd == FRHIP_F32 && dd == FRHIP_F16)
    hipLaunchKernelGGL((cast_kernel<float, h1>), dim3(blocks_for(n, 256)), dim3(256), 0, st, (const float*)src, (h1*)dst, n);
  else if (sd == dd && (sd == FRHIP_F16 || sd == FRHIP_F32))
    return hip_result(hipMemcpyAsync(dst, src, n * (sd == FRHIP_F16 ? 2 : 4), hipMemcpyDeviceToDevice, st), "cast copy");
  else
    return set_error(FRHIP_EINVAL, "cast: unsupported dtype pair");
  return check_launch("cast");
}

int frhip_fill(void* x, int dtype, float value, size_t n, frhip_stream s) {
  if (!x) return set_error(FRHIP_EINVAL, "fill: null pointer");
  if (n == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  if (dtype == FRHIP_F16)
    hipLaunchKernelGGL(fill_kernel<h1>, dim3(blocks_for(n, 256)), dim3(256), 0, st, (h1*)x, (h1)value, n);
  else if (dtype == FRHIP_F32)
    hipLaunchKernelGGL(fill_kernel<float>, dim3(blocks_for(n, 256)), dim3(256), 0, st, (float*)x, value, n);
  else if (dtype == FRHIP_U8)
    hipLaunchKernelGGL(fill_kernel<unsigned char>, dim3(blocks_for(n, 256)), dim3(256), 0, st, (unsigned char*)x,
                       (unsigned char)value, n);
  else
    return set_error(FRHIP_EINVAL, "fill: unknown dtype");
  return check_launch("fill");
}

int frhip_scalar_div_f16(void* x, float divisor, size_t n, frhip_stream s) {
  if (!x) return set_error(FRHIP_EINVAL, "scalar_div: null pointer");
  if (n == 0) return 0;
  hipLaunchKernelGGL(scalar_div_f16_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, static_cast<hipStream_t>(s), (h1*)x,
                     (h1)divisor, n);
  return check_launch("scalar_div");
}

int frhip_gather_rows(const void* table, const int32_t* ids_dev, void* out, int n_ids, int row_bytes, frhip_stream s) {
  if (!table || !ids_dev || !out) return set_error(FRHIP_EINVAL, "gather: null pointer");
  if (n_ids < 0 || row_bytes <= 0 || row_bytes % 16 != 0) return set_error(FRHIP_ESHAPE, "gather: row_bytes must be a multiple of 16");
  if (n_ids == 0) return 0;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n_ids), dim3(256), 0, static_cast<hipStream_t>(s),
                     (const unsigned char*)table, ids_dev, (unsigned char*)out, row_bytes);
  return check_launch("gather_rows");
}

int frhip_embed_ring(const void* table, int n_rows, int row_bytes, const int32_t* ring, int ring_len,
                     uint32_t* counter_dev, void* out, frhip_stream s) {
  if (!table || !ring || !counter_dev || !out) return set_error(FRHIP_EINVAL, "embed_ring: null pointer");
  if (n_rows <= 0 || ring_len <= 0 || row_bytes <= 0 || row_bytes % 16 != 0)
    return set_error(FRHIP_ESHAPE, "embed_ring: row_bytes must be a positive multiple of 16");
  hipLaunchKernelGGL(embed_ring_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(s),
                     (const unsigned char*)table, n_rows, row_bytes, ring, ring_len, counter_dev, (unsigned char*)out);
  return check_launch("embed_ring");
}

int frhip_embed_argmax(const void* table, int n_rows, int row_bytes, const void* pairs, int npairs, int32_t* ids,
                       int ids_len, uint32_t* counter_dev, void* out, frhip_stream s) {
  if (!table || !pairs || !ids || !counter_dev || !out) return set_error(FRHIP_EINVAL, "embed_argmax: null pointer");
  if (n_rows <= 0 || npairs <= 0 || ids_len <= 0 || row_bytes <= 0 || row_bytes % 16 != 0)
    return set_error(FRHIP_ESHAPE, "embed_argmax: row_bytes must be a positive multiple of 16");
  hipLaunchKernelGGL(embed_argmax_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(s), (const unsigned char*)table,
                     n_rows, row_bytes, (const float*)pairs, npairs, ids, ids_len, counter_dev, (unsigned char*)out);
  return check_launch("embed_argmax");
}

int frhip_pack_transpose(const void* src, void* dst, int K, int N, int elem_bytes, frhip_stream s) {
  if (!src || !dst) return set_error(FRHIP_EINVAL, "pack: null pointer");
  if (K <= 0 || N <= 0) return set_error(FRHIP_ESHAPE, "pack: empty matrix");
  dim3 grid((N + 63) / 64, (K + 63) / 64);
  hipStream_t st = static_cast<hipStream_t>(s);
  if (elem_bytes == 2)
    hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, st, (const uint16_t*)src, (uint16_t*)dst, K, N);
  else if (elem_bytes == 1)
    hipLaunchKernelGGL(transpose_kernel<uint8_t>, grid, dim3(256), 0, st, (const uint8_t*)src, (uint8_t*)dst, K, N);
  else
    return set_error(FRHIP_EINVAL, "pack: elem_bytes must be 1 or 2");
  return check_launch("pack_transpose");
}

int frhip_dequant_u8(const frhip_weight* w, void* dst, frhip_stream s) {
  if (!w || !w->data || !dst) return set_error(FRHIP_EINVAL, "dequant: null pointer");
  if (w->dtype != FRHIP_U8 || !w->mx || !w->rx || !w->my || !w->ry) return set_error(FRHIP_EINVAL, "dequant: not a uint8 weight");
  if (w->K <= 0 || w->N <= 0 || w->K % 4 != 0) return set_error(FRHIP_ESHAPE, "dequant: K must be a multiple of 4");
  return dequant_u8_async((const unsigned char*)w->data, (const h1*)w->mx, (const h1*)w->rx, (const h1*)w->my,
                          (const h1*)w->ry, (h1*)dst, w->K, w->N, static_cast<hipStream_t>(s));
}

int frhip_copy_probe(void* dst, const void* src, size_t bytes, frhip_stream s) {
  if (!dst || !src) return set_error(FRHIP_EINVAL, "copy_probe: null pointer");
  if (bytes % 16 != 0) return set_error(FRHIP_ESHAPE, "copy_probe: bytes must be a multiple of 16");
  if (bytes == 0) return 0;
  hipLaunchKernelGGL(copy_probe_kernel, dim3(compute_units() * 8), dim3(256), 0, static_cast<hipStream_t>(s),
                     (const u32x4*)src, (u32x4*)dst, bytes / 16);
  return check_launch("copy_probe");
}

int frhip_read_probe(const void* src, size_t bytes, void* sink, frhip_stream s) {
  if (!src || !sink) return set_error(FRHIP_EINVAL, "read_probe: null pointer");
  if (bytes % 16 != 0) return set_error(FRHIP_ESHAPE, "read_probe: bytes must be a multiple of 16");
  if (bytes == 0) return 0;
  int grid = compute_units() * 2;
  if (grid > 2048) grid = 2048;
  hipLaunchKernelGGL(read_probe_kernel, dim3(grid), dim3(512), 0, static_cast<hipStream_t>(s), (const u32x4*)src,
                     bytes / 16, (uint32_t*)sink);
  return check_launch("read_probe");
}

int frhip_argmax_blocks_f32_mirror(const float* x, int n, void* pairs, void* mirror, int nblocks, frhip_stream s) {
  if (!x || !pairs) return set_error(FRHIP_EINVAL, "argmax: null pointer");
  if (n <= 0 || nblocks <= 0) return set_error(FRHIP_ESHAPE, "argmax: empty input");
  if (reinterpret_cast<uintptr_t>(x) % 16) return set_error(FRHIP_EINVAL, "argmax: x must be 16-byte aligned");
  const int len = ((n + nblocks - 1) / nblocks + 3) / 4 * 4;
  hipLaunchKernelGGL(argmax_blocks_f32_kernel, dim3(nblocks), dim3(256), 0, static_cast<hipStream_t>(s), x, n, len,
                     static_cast<float*>(pairs), static_cast<float*>(mirror));
  return check_launch("argmax_blocks");
}

int frhip_argmax_blocks_f32(const float* x, int n, void* pairs, int nblocks, frhip_stream s) {
  return frhip_argmax_blocks_f32_mirror(x, n, pairs, nullptr, nblocks, s);
}

int frhip_argmax_f32(const float* logits, int n, int32_t* out_id, frhip_stream s) {
  if (!logits || !out_id) return set_error(FRHIP_EINVAL, "argmax: null pointer");
  if (n <= 0) return set_error(FRHIP_ESHAPE, "argmax: empty input");
  hipLaunchKernelGGL(argmax_f32_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(s), logits, n, out_id);
  return check_launch("argmax");
}

int frhip_slice(const void* src, void* dst, int ndim, const int* src_shape, const int* start, const int* interval,
                const int* dst_shape, int elem_bytes, frhip_stream s) {
  if (!src || !dst) return set_error(FRHIP_EINVAL, "slice: null pointer");
  Dims4 ss, ds, st4, iv;
  if (!to_dims4(src_shape, ndim, 1, &ss) || !to_dims4(dst_shape, ndim, 1, &ds) || !to_dims4(start, ndim, 0, &st4) ||
      !to_dims4(interval, ndim, 1, &iv))
    return set_error(FRHIP_ESHAPE, "slice: 1 to 4 dimensions");
  size_t total = 1;
  for (int d = 0; d < 4; d++) {
    if (ss.n[d] <= 0 || ds.n[d] < 0 || st4.n[d] < 0 || iv.n[d] <= 0) return set_error(FRHIP_ESHAPE, "slice: bad range");
    if (ds.n[d] > 0 && (long)st4.n[d] + (long)(ds.n[d] - 1) * iv.n[d] >= ss.n[d])
      return set_error(FRHIP_ESHAPE, "slice: range runs past the source dimension");
    total *= (size_t)ds.n[d];
  }
  if (total == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  int rc = by_elem_bytes(elem_bytes, [&](auto tag) {
    using T = decltype(tag);
    hipLaunchKernelGGL(slice_kernel<T>, dim3(blocks_for(total, 256)), dim3(256), 0, st, (const T*)src, (T*)dst, ss, ds, st4,
                       iv, total);
  });
  return rc ? rc : check_launch("slice");
}

int frhip_cat(const void* a, const void* b, void* out, size_t left, size_t a_mid, size_t b_mid, size_t right,
              int elem_bytes, frhip_stream s) {
  if (!a || !b || !out) return set_error(FRHIP_EINVAL, "cat: null pointer");
  const size_t total = left * (a_mid + b_mid) * right;
  if (total == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  int rc = by_elem_bytes(elem_bytes, [&](auto tag) {
    using T = decltype(tag);
    hipLaunchKernelGGL(cat_kernel<T>, dim3(blocks_for(total, 256)), dim3(256), 0, st, (const T*)a, (const T*)b, (T*)out,
                       a_mid, b_mid, right, total);
  });
  return rc ? rc : check_launch("cat");
}

int frhip_transpose(const void* src, void* dst, int ndim, const int* shape, int dim_a, int dim_b, int elem_bytes,
                    frhip_stream s) {
  if (!src || !dst) return set_error(FRHIP_EINVAL, "transpose: null pointer");
  Dims4 ss;
  if (!to_dims4(shape, ndim, 1, &ss)) return set_error(FRHIP_ESHAPE, "transpose: 1 to 4 dimensions");
  if (dim_a < 0 || dim_b < 0 || dim_a >= ndim || dim_b >= ndim) return set_error(FRHIP_EINVAL, "transpose: dimension out of range");
  size_t total = 1;
  for (int d = 0; d < 4; d++) {
    if (ss.n[d] <= 0) return set_error(FRHIP_ESHAPE, "transpose: empty dimension");
    total *= (size_t)ss.n[d];
  }
  hipStream_t st = static_cast<hipStream_t>(s);
  int rc = by_elem_bytes(elem_bytes, [&](auto tag) {
    using T = decltype(tag);
    hipLaunchKernelGGL(transpose_nd_kernel<T>, dim3(blocks_for(total, 256)), dim3(256), 0, st, (const T*)src, (T*)dst, ss,
                       dim_a + 4 - ndim, dim_b + 4 - ndim, total);
  });
  return rc ? rc : check_launch("transpose");
}

int frhip_silu(const void* x, void* y, int dtype, size_t n, frhip_stream s) {
  if (!x || !y) return set_error(FRHIP_EINVAL, "silu: null pointer");
  if (n == 0) return 0;
  hipStream_t st = static_cast<hipStream_t>(s);
  if (dtype == FRHIP_F16)
    hipLaunchKernelGGL(silu_f16_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, st, (const h1*)x, (h1*)y, n);
  else if (dtype == FRHIP_F32)
    hipLaunchKernelGGL(silu_f32_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, st, (const float*)x, (float*)y, n);
  else
    return set_error(FRHIP_EINVAL, "silu: dtype must be F16 or F32");
  return check_launch("silu");
}

int frhip_mfma_probe(int waves_per_workgroup, int iters, const void* operands, void* sink, void* clocks, frhip_stream s) {
  if (!operands || !sink || !clocks) return set_error(FRHIP_EINVAL, "mfma_probe: null pointer");
  if (waves_per_workgroup < 1 || waves_per_workgroup > 8 || iters < 1) return set_error(FRHIP_EINVAL, "mfma_probe: 1..8 waves, iters >= 1");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(compute_units()), dim3(waves_per_workgroup * kWave), 0, static_cast<hipStream_t>(s),
                     (const h8*)operands, iters, (float*)sink, (unsigned long long*)clocks);
  return check_launch("mfma_probe");
}

}  // extern "C"
