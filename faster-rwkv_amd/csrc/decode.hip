// One-token (batch-1 decode) kernels for gfx950.
//
// The decode step of RWKV is a chain of matrix-vector products separated by cheap
// elementwise work; each product streams its weight matrix from HBM exactly once,
// so the whole step is bound by HBM bandwidth and, because a 2048x2048 binary16
// matrix is only 8 MB (1 us at 8 TB/s), by how fast a launch gets its loads in flight.
// The kernels are organised around that:
//   * weights are output-major ([N][K]); a wavefront takes whole rows, each lane
//     loads 16 contiguous bytes per row chunk, products accumulate in fp32 and are
//     reduced across lanes with DPP adds.  No partial sums ever leave the wave, so
//     every elementwise epilogue (sigmoid, WKV update, relu^2, residual) runs in
//     the lane that owns the output and is fused into the same launch;
//   * a wave issues the loads of its first batch of rows BEFORE the workgroup's
//     prologue (weights do not depend on activations), so HBM latency overlaps the
//     layernorm / token-shift work; with one workgroup per CU most launches are a
//     single batch per wave, i.e. the whole matrix is requested in the first microsecond;
//   * the layernorm + token-shift mix that precedes a product is recomputed by
//     every workgroup into LDS (the activation vector is a few KB and L2-resident),
//     which removes the separate launches the reference makes for them
//     (kernels/cuda/att.cu:183-188, ffn.cu:66-75);
//   * independent products share a launch (key/value/receptance of att; receptance
//     and key of ffn) so that a launch moves tens of MB.
// One RWKV-4 layer is four launches; the reference issues seventeen
// (kernels/cuda/att.cu:182-217, ffn.cu:62-87).
#include <climits>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "device_utils.h"
#include "frhip_internal.h"

#pragma clang fp contract(off)

namespace frhip {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;

// Measurement build (`make timeline` -> -DFRHIP_TIMELINE, a library of its own): every wave of rows_kernel notes the
// 100 MHz clock at the points marked FR_TL(i), keeps the notes in registers and leaves them in g_timeline[slot][wave]
// when it ends (so the notes add no memory operation before the kernel's last store); launches take the slots round
// robin; frhip_timeline_read copies them out.  Compiled out otherwise.
#ifdef FRHIP_TIMELINE
constexpr int kTlStamps = 16, kTlSlots = 8, kTlWaves = 4096;
__device__ unsigned long long g_timeline[kTlSlots][kTlWaves][kTlStamps];
static int g_timeline_launches = 0;
#define FR_TL_DECL unsigned long long fr_tl[kTlStamps] = {}
#define FR_TL(i) fr_tl[i] = __builtin_amdgcn_s_memrealtime()
#define FR_TL_AFTER(i, v)            \
  do {                               \
    asm volatile("" ::"v"(v));       \
    FR_TL(i);                        \
  } while (0)
#define FR_TL_FLUSH(slot)                                                                            \
  do {                                                                                               \
    __builtin_amdgcn_s_waitcnt(0);                                                                   \
    FR_TL(kTlStamps - 1);                                                                            \
    const int fr_w = (int)blockIdx.x * kWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave); \
    if ((threadIdx.x & (kWave - 1)) == 0 && fr_w < kTlWaves) {                                       \
      for (int fr_i = 0; fr_i < kTlStamps; fr_i++) g_timeline[slot][fr_w][fr_i] = fr_tl[fr_i];      \
    }                                                                                                \
  } while (0)
#else
#define FR_TL_DECL
#define FR_TL(i)
#define FR_TL_AFTER(i, v)
#define FR_TL_FLUSH(slot)
#endif
constexpr int kMaxSeg = 4;
constexpr int kFusedMaxC = 8 * kThreads;  // widest vector the fused layernorm prologues take
constexpr int kMaxC = 16384;

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

// `red` holds 2 * kWaves floats: the two reductions use separate halves, one barrier each.
// The thread's eight elements and their gamma / beta arrive in registers: callers request them
// ahead of the weight rows, so that the normalisation runs while the rows are in flight
// (vector loads return in the order they were issued).
__device__ __forceinline__ LnOut ln_regs(h8 xv, h8 g, h8 b, bool active, int C, float* red) {
  LnOut o;
  o.active = active;
  float xf[8];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    xf[i] = active ? (float)xv[i] : 0.f;
    s += xf[i];
  }
  const float mean = block_sum1<kWaves>(s, red) / (float)C;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    float d = xf[i] - mean;
    q += active ? d * d : 0.f;
  }
  float var = block_sum1<kWaves>(q, red + kWaves) / (float)C;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    h1 n = (h1)((xf[i] - mean) * inv);
    o.xx[i] = (n * g[i]) + b[i];
  }
  return o;
}

__device__ __forceinline__ h8 mix8(h8 xx, h8 sx, h8 m) {
  h8 o;
#pragma unroll
  for (int i = 0; i < 8; i++) o[i] = mix1(xx[i], sx[i], m[i]);
  return o;
}

// Even split of items over the waves of the grid with the division done on the host:
// wave i gets `base` items, the first `rem` waves one more.
struct Split {
  int base, rem;
};

// Index of this wave among the waves of the grid, for dealing out work with split_even.  Where the
// items do not divide evenly the first `rem` indices get one more: numbering the waves across the
// workgroups first (wave 0 of every workgroup, then wave 1 of every workgroup, ...) spreads those
// over all compute units instead of loading the first ones with eight longer waves each and leaving
// the last ones short (ffn_front of the 1.5B shape, 1708 batches for 2048 waves: 10.2 -> 9.4 us).
// An even split keeps neighbouring rows in neighbouring waves of one workgroup (att_out: 3.6 us
// against 3.8 us numbered the other way).
__device__ __forceinline__ int grid_wave(Split sp) {
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  return sp.rem != 0 ? wv * (int)gridDim.x + (int)blockIdx.x : (int)blockIdx.x * kWaves + wv;
}

__device__ __forceinline__ void split_even(Split sp, int i, int& lo, int& hi) {
  lo = i * sp.base + (i < sp.rem ? i : sp.rem);
  hi = lo + sp.base + (i < sp.rem ? 1 : 0);
}

// ---------------------------------------------------------------------------
// A batch of R weight rows held in registers: NCH 16-byte chunks per lane per row
// (lane l owns chunks l, l+64, ...).  load() only issues the loads; dot() consumes
// them against LDS-resident vectors.  K <= NCH * 64 * (8 | 16) elements.
// Neither contains a branch, so that the compiler can count the loads in flight and let
// dot() start on the first chunk while later ones (and the next batch) are still on their
// way: a lane whose chunk index lies beyond the row re-reads the row's last chunk, and the
// staged vectors are padded with zeros up to NCH * 64 chunks, which cancels it.
// ---------------------------------------------------------------------------
template <int R, int NCH, bool U8>
struct RowBatch {
  using V = typename std::conditional<U8, u32x4, h8>::type;
  static constexpr int kPadChunks = NCH * kWave;  // chunks per staged vector, padding included
  V w[R][NCH];

  // Rows are read through buffer descriptors (base = start of the row, extent = nbytes[r]): a
  // lane whose chunk lies beyond the extent gets zeros without a memory access, which serves
  // the tail of a row whose length is not a multiple of 64 chunks, the surplus slots of a short
  // batch and waves without work (extent 0) alike, with the same number of loads issued.
  template <int J0 = 0, int J1 = NCH>
  __device__ __forceinline__ void load(const void* const (&rows)[R], const int (&nbytes)[R], int lane) {
    __amdgpu_buffer_rsrc_t rs[R];
#pragma unroll
    for (int r = 0; r < R; r++)
      rs[r] = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(rows[r]), 0, nbytes[r], 0x00020000);
    // chunk-major, the order in which dot_shared() consumes them; chunks J0 .. J1-1 only
#pragma unroll
    for (int j = J0; j < J1; j++) {
#pragma unroll
      for (int r = 0; r < R; r++) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs[r], lane * 16 + (j & 3) * (kWave * 16),
                                                              (j >> 2) * (4 * kWave * 16), 2 /* nontemporal */);
        w[r][j] = __builtin_bit_cast(V, v);
      }
    }
  }

  // The same for a slice of rows longer than one register tiling: chunk j of the slice lies `sbase`
  // bytes + (j * 64 + lane) chunks into the row.  The slice's byte offset goes into the scalar offset
  // of the load, and the extents passed in end where the slice ends, so chunks of the tiling that the
  // slice does not use read zeros without a memory access, like any other tail.
  __device__ __forceinline__ void load_slice(const void* const (&rows)[R], const int (&nbytes)[R], int lane, int sbase) {
    __amdgpu_buffer_rsrc_t rs[R];
#pragma unroll
    for (int r = 0; r < R; r++)
      rs[r] = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(rows[r]), 0, nbytes[r], 0x00020000);
#pragma unroll
    for (int j = 0; j < NCH; j++) {
#pragma unroll
      for (int r = 0; r < R; r++) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs[r], lane * 16 + (j & 3) * (kWave * 16),
                                                              sbase + (j >> 2) * (4 * kWave * 16), 2 /* nontemporal */);
        w[r][j] = __builtin_bit_cast(V, v);
      }
    }
  }

  // Chunks of a batch requested ahead of the prologue.  A compute unit keeps only so many bytes of
  // loads in flight (about 64 KB: 8 per wave); a wave that asks for more is held at the load
  // instruction until earlier data has returned, and the older four waves of a workgroup go first.
  // A prologue that sits behind all loads of a large batch therefore runs when most rows have
  // arrived (its barriers wait for the last wave to get through its loads).  Batches of more than
  // 16 loads put about 8 of them first, then the prologue, then the rest; for smaller ones holding
  // loads back only idles the memory (measured: 24 loads, 6 first: 9.60 -> 9.33 us; 16 loads, 8
  // first: 7.11 -> 7.32 us; 12 loads, 6 first: 6.81 -> 7.12 us).
  // uint8 rows cost two VALU operations per code, about as long as their bytes take to arrive: the
  // sooner the prologue's barrier, the more of the products run under the stream, so only about
  // six loads go first there.
  // (uint8, re-measured as decode tok/s of the 1.5B RWKV-4 / 8 layers of the 3B RWKV-5.2: about 6 loads first
  // 1576 / 2808, about 12 first -- the whole batch of the 1.5B shape -- 1515 / 2793, the whole batch of the 3B shape 2686;
  // binary16: whole batches first 1407 / 2539 against 1445 / 2628 as below, 12 first 1401 / 2628.)
  static constexpr int kFirst = U8 ? 6 : 8;
  static constexpr int kHead0 = R * NCH <= (U8 ? 6 : 16) ? NCH : (kFirst / R < 1 ? 1 : kFirst / R);
  static constexpr int kHead = kHead0 < NCH ? kHead0 : NCH;  // never beyond the batch

  // All rows against one staged vector, each chunk of which is read from LDS once.  Binary16 rows:
  // acc[r] = sum_k w[k] x[k] against a binary16 vector; uint8 rows: acc[r] = sum_k q[k] xr[k]
  // against an fp32 vector staged by stage_q.
  __device__ __forceinline__ void dot_shared(const void* xv, int lane, float (&acc)[R]) const {
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    dot_add(xv, lane, 0, kPadChunks, acc);
  }

  // acc[r] += the products of this batch against chunks c0 + lane + j * 64 of a staged vector of
  // `padchunks` chunks (the stride between the four 16-byte groups of a uint8 chunk).
  __device__ __forceinline__ void dot_add(const void* xv, int lane, int c0, int padchunks, float (&acc)[R]) const {
#pragma unroll
    for (int j = 0; j < NCH; j++) {
      const int c = c0 + lane + j * kWave;
      if constexpr (!U8) {
        const h8 x = reinterpret_cast<const h8*>(xv)[c];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = dot8acc(w[r][j], x, acc[r]);
      } else {
        const f32x4* xp = reinterpret_cast<const f32x4*>(xv) + c;
        float e[R], o[R];
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = o[r] = 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
          const f32x4 x = xp[jj * padchunks];
#pragma unroll
          for (int r = 0; r < R; r++) {
            const uint32_t word = w[r][j][jj];
            e[r] = __builtin_fmaf((float)(word & 0xffu), x[0], e[r]);
            o[r] = __builtin_fmaf((float)((word >> 8) & 0xffu), x[1], o[r]);
            e[r] = __builtin_fmaf((float)((word >> 16) & 0xffu), x[2], e[r]);
            o[r] = __builtin_fmaf((float)(word >> 24), x[3], o[r]);
          }
        }
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] += e[r] + o[r];
      }
    }
  }

};

// Bytes of LDS one staged vector takes for a given tiling (padding included).
__host__ __device__ constexpr size_t staged_bytes(int nch, bool u8) { return (size_t)nch * kWave * (u8 ? 64 : 16); }

// Zero the padding chunks [nchunk, padchunks) of a staged vector.
template <bool U8>
__device__ __forceinline__ void zero_pad(void* vec, int nchunk, int padchunks) {
  for (int c = nchunk + (int)threadIdx.x; c < padchunks; c += kThreads) {
    if constexpr (!U8) {
      reinterpret_cast<h8*>(vec)[c] = h8{};
    } else {
#pragma unroll
      for (int jj = 0; jj < 4; jj++) reinterpret_cast<f32x4*>(vec)[jj * padchunks + c] = f32x4{};
    }
  }
}

// ---------------------------------------------------------------------------
// uint8 matrices in the row-streaming kernels.  With w^[n][k] = q c_n ry_k + mx_n + my_k
// (c_n = rx_n / 255) a row's product factors into
//   sum_k x_k w^[n][k] = c_n sum_k (x_k ry_k) q[n][k] + mx_n sum_k x_k + sum_k x_k my_k ,
// so only the first sum depends on the row.  The workgroup stages xr_k = x_k ry_k in fp32 (the
// product of two binary16 values is exact there) once per matrix and reduces Sx = sum x and
// Smy = sum x my; a row then costs one byte-to-float conversion and one fma per code and
// finishes as  c_n D_n + mx_n Sx + Smy.  This is the dequantisation formula evaluated in fp32
// without its final rounding of w^ to binary16 (which the standalone dequantisation and the
// matrix-matrix kernel apply); the difference is below the rounding of the binary16 output.
//
// xr is staged "split": a lane's chunk c covers 16 codes = four 16-byte groups of xr, and
// group j of chunk c lives at f32x4 index j * padchunks + c, so that consecutive lanes read
// consecutive 16-byte LDS words.
// ---------------------------------------------------------------------------
constexpr int kQSums = 2;  // Sx, Smy

// Thread-owned group g = 8 consecutive elements of the vector: xr = x * ry into the staged vector.
__device__ __forceinline__ void stage_xr(float* dst, int g, int padchunks, h8 x, h8 ry) {
  const int nchunk = padchunks;
  f32x4 lo, hi;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    lo[i] = (float)x[i] * (float)ry[i];
    hi[i] = (float)x[4 + i] * (float)ry[4 + i];
  }
  const int c = g >> 1, j = (g & 1) * 2;
  reinterpret_cast<f32x4*>(dst)[j * nchunk + c] = lo;
  reinterpret_cast<f32x4*>(dst)[(j + 1) * nchunk + c] = hi;
}

// The group's share of Sx = sum x and Smy = sum x my, with the packed dot product (products of two
// binary16 values are exact in fp32): 8 instructions instead of 32 conversions, adds and fmas.
__device__ __forceinline__ void sum_q(h8 x, h8 my, float* part) {
  h8 ones;
#pragma unroll
  for (int i = 0; i < 8; i++) ones[i] = (h1)1.0f;
  part[0] = dot8acc(x, ones, part[0]);
  part[1] = dot8acc(x, my, part[1]);
}

__device__ __forceinline__ void stage_q(float* dst, int g, int padchunks, h8 x, h8 ry, h8 my, float* part) {
  stage_xr(dst, g, padchunks, x, ry);
  sum_q(x, my, part);
}

// Per-wave sums of the nval per-thread partials go to red[wave][v]; the caller's next barrier
// publishes them, after which lane v of every wave gathers total v with gather_qsums.
__device__ __forceinline__ void publish_qsums(const float* part, int nval, float (*red)[kMaxSeg * kQSums]) {
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  for (int v = 0; v < nval; v++) {
    const float t = wave_sum(part[v]);
    if (lane == 0) red[wv][v] = t;
  }
}

__device__ __forceinline__ float gather_qsums(int nval, const float (*red)[kMaxSeg * kQSums]) {
  const int lane = threadIdx.x & (kWave - 1);
  float t = 0.f;
  if (lane < nval) {
#pragma unroll
    for (int i = 0; i < kWaves; i++) t += red[i][lane];
  }
  return t;
}

__device__ __forceinline__ float finish_q(float d, float rx, float mx, float sx, float smy) {
  const float c = rx / 255.0f;
  return c * d + mx * sx + smy;
}

// ===========================================================================
// att, front half:  LN -> mix -> k,v,r products -> sigmoid -> WKV-4 update
//                   -> r * wkv                    (kernels/cuda/att.cu:183-211)
// One channel = three rows (one of each matrix); the wave that owns a channel owns
// its recurrent state.
// ===========================================================================
struct AttFrontV4 {
  int C;
  Split split;  // channels over the waves of the grid
  const h1 *x, *sx, *ln_w, *ln_b, *mk, *mv, *mr;
  const float *aa, *bb, *pp, *td, *tf;
  WMat kw, vw, rw;
  h1 *xx_out, *rwkv_out;
  float *aa_out, *bb_out, *pp_out;
};

// SINGLE: no wave owns more than one channel (the host checks).  That kernel has no loop and no
// second set of rows, so nothing competes with the loads in flight for registers.
template <int NCH, bool U8, bool SINGLE>
__global__ __launch_bounds__(kThreads) void att_front_v4_kernel(AttFrontV4 a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[2 * kWaves];
  // One field from every 64-byte line of the kernel arguments is requested up front, so that the
  // scalar loads further down (issued where each field is first needed) hit the scalar cache.
  asm volatile("" ::"s"(a.C), "s"(a.tf), "s"(a.vw.data), "s"(a.rw.data), "s"(a.xx_out));
  const int C = a.C;
  const int nchunk = U8 ? (C >> 4) : (C >> 3);
  // binary16: the three mixed vectors; uint8: the three pre-scaled fp32 vectors xr (see stage_q)
  constexpr int kPad = NCH * kWave;
  constexpr size_t kVecBytes = staged_bytes(NCH, U8);
  unsigned char* kx = smem;
  unsigned char* vx = kx + kVecBytes;
  unsigned char* rx = vx + kVecBytes;
  __shared__ float qred[kWaves][kMaxSeg * kQSums];

  const int lane = threadIdx.x & (kWave - 1);
  // wave-uniform, and known to the compiler as such: row addresses stay in scalar registers
  const int gw = grid_wave(a.split);
  int c0, c1;
  split_even(a.split, gw, c0, c1);
  const size_t row_bytes = U8 ? (size_t)C : 2 * (size_t)C;

  // the three rows of a channel as three one-row batches: each multiplies its own staged vector
  struct Rows3 {
    RowBatch<1, NCH, U8> k, v, r;
  };
  // chunks J0 .. J1-1 of the three rows of channel n
  auto load3_part = [&](Rows3& b, int n, bool live, auto j0, auto j1) {
    const void* rk[1] = {a.kw.data + n * row_bytes};
    const void* rv[1] = {a.vw.data + n * row_bytes};
    const void* rr[1] = {a.rw.data + n * row_bytes};
    const int nb[1] = {live ? (int)row_bytes : 0};
    b.k.template load<decltype(j0)::value, decltype(j1)::value>(rk, nb, lane);
    b.v.template load<decltype(j0)::value, decltype(j1)::value>(rv, nb, lane);
    b.r.template load<decltype(j0)::value, decltype(j1)::value>(rr, nb, lane);
  };
  using J0 = std::integral_constant<int, 0>;
  // requested ahead of the prologue: uint8, one chunk of each row (its products take as long as its bytes)
  using JH = std::integral_constant<int, U8 ? 1 : RowBatch<3, NCH, U8>::kHead>;
  using JN = std::integral_constant<int, NCH>;
  auto load3 = [&](Rows3& b, int n, bool live) { load3_part(b, n, live, J0{}, JN{}); };
  // Every global operand is requested before the first wait, operands of the prologue first: the
  // layernorm and the staging then run while the weight rows are in flight, and the products
  // start on the first chunks that arrive (vector loads return in the order they were issued).
  // The rows are loaded unconditionally and last (waves without a channel read a valid
  // duplicate): a load inside a branch after them would make the number of loads in flight
  // path-dependent and every later wait a wait for all of them.  Before them branches are
  // harmless, and only threads that own a group load: every byte requested here passes through
  // the compute unit's vector memory pipeline ahead of the rows.
  const bool own = (int)threadIdx.x * 8 < C;
  const int e0 = threadIdx.x * 8;
  h8 xv{}, lg{}, lb{}, sx{}, mixk{}, mixv{}, mixr{}, qry[3] = {}, qmy[3] = {};
  if (own) {
    xv = *reinterpret_cast<const h8*>(a.x + e0);
    lg = *reinterpret_cast<const h8*>(a.ln_w + e0);
    lb = *reinterpret_cast<const h8*>(a.ln_b + e0);
    sx = *reinterpret_cast<const h8*>(a.sx + e0);
    mixk = *reinterpret_cast<const h8*>(a.mk + e0);
    mixv = *reinterpret_cast<const h8*>(a.mv + e0);
    mixr = *reinterpret_cast<const h8*>(a.mr + e0);
    if constexpr (U8) {
      qry[0] = *reinterpret_cast<const h8*>(a.kw.ry + e0); qmy[0] = *reinterpret_cast<const h8*>(a.kw.my + e0);
      qry[1] = *reinterpret_cast<const h8*>(a.vw.ry + e0); qmy[1] = *reinterpret_cast<const h8*>(a.vw.my + e0);
      qry[2] = *reinterpret_cast<const h8*>(a.rw.ry + e0); qmy[2] = *reinterpret_cast<const h8*>(a.rw.my + e0);
    }
  }
  // recurrent state and per-row constants of a channel (every lane reads the same words)
  struct Chan {
    float tf, td, pp, aa, bb;
    h1 qrx[3], qmx[3];
  };
  auto load_chan = [&](Chan& s, int n) {
    s.tf = a.tf[n]; s.td = a.td[n]; s.pp = a.pp[n]; s.aa = a.aa[n]; s.bb = a.bb[n];
    if constexpr (U8) {
      s.qrx[0] = a.kw.rx[n]; s.qmx[0] = a.kw.mx[n];
      s.qrx[1] = a.vw.rx[n]; s.qmx[1] = a.vw.mx[n];
      s.qrx[2] = a.rw.rx[n]; s.qmx[2] = a.rw.mx[n];
    }
  };
  Rows3 cur;
  Chan st;
  {
    const int first = c0 < c1 ? c0 : C - 1;
    load_chan(st, first);
    load3_part(cur, first, c0 < c1, J0{}, JH{});
  }

  LnOut ln = ln_regs(xv, lg, lb, own, C, red);
  float part[3 * kQSums];
#pragma unroll
  for (int i = 0; i < 3 * kQSums; i++) part[i] = 0.f;
  h8 mk{}, mv{}, mr{};
  if (ln.active) {
    mk = mix8(ln.xx, sx, mixk);
    mv = mix8(ln.xx, sx, mixv);
    mr = mix8(ln.xx, sx, mixr);
    if constexpr (U8) {
      stage_xr(reinterpret_cast<float*>(kx), threadIdx.x, kPad, mk, qry[0]);
      stage_xr(reinterpret_cast<float*>(vx), threadIdx.x, kPad, mv, qry[1]);
      stage_xr(reinterpret_cast<float*>(rx), threadIdx.x, kPad, mr, qry[2]);
    } else {
      reinterpret_cast<h8*>(kx)[threadIdx.x] = mk;
      reinterpret_cast<h8*>(vx)[threadIdx.x] = mv;
      reinterpret_cast<h8*>(rx)[threadIdx.x] = mr;
    }
    if (blockIdx.x == 0) *reinterpret_cast<h8*>(a.xx_out + e0) = ln.xx;
  }
  zero_pad<U8>(kx, nchunk, kPad);
  zero_pad<U8>(vx, nchunk, kPad);
  zero_pad<U8>(rx, nchunk, kPad);
  __syncthreads();
  load3_part(cur, c0 < c1 ? c0 : C - 1, c0 < c1, JH{}, JN{});  // the rest of the first channel's rows
  float qt[3 * kQSums];
  if constexpr (U8) {
    // Sx and Smy of the three vectors are needed only when a row is finished: they are summed here, behind the
    // barrier that releases the staged vectors and behind the last row requests, while the rows are on their way
    // (every thread reaches both barriers; a thread without a group adds zeros).
    sum_q(mk, qmy[0], part + 0 * kQSums);
    sum_q(mv, qmy[1], part + 1 * kQSums);
    sum_q(mr, qmy[2], part + 2 * kQSums);
    publish_qsums(part, 3 * kQSums, qred);
    __syncthreads();
    const float tv = gather_qsums(3 * kQSums, qred);
#pragma unroll
    for (int i = 0; i < 3 * kQSums; i++) qt[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tv), i));
  }

  // products, reduction and state update of one channel whose rows and state are in registers
  auto channel = [&](int n, const Rows3& rows, const Chan& st) {
    float acc[3];
    {
      float t[1];
      rows.k.dot_shared(kx, lane, t);
      acc[0] = t[0];
      rows.v.dot_shared(vx, lane, t);
      acc[1] = t[0];
      rows.r.dot_shared(rx, lane, t);
      acc[2] = t[0];
    }
    float k = wave_sum(acc[0]);
    float v = wave_sum(acc[1]);
    float rr = wave_sum(acc[2]);
    if constexpr (U8) {
      k = finish_q(k, (float)st.qrx[0], (float)st.qmx[0], qt[0], qt[1]);
      v = finish_q(v, (float)st.qrx[1], (float)st.qmx[1], qt[2], qt[3]);
      rr = finish_q(rr, (float)st.qrx[2], (float)st.qmx[2], qt[4], qt[5]);
    }
    // kernels/cuda/att.cu:30-62 (WkvForwardOne), r already passed through sigmoid (:203).
    // The update is a chain of five exponentials and two quotients on one channel's scalars, at the very end of
    // the launch.  Every lane holds k, v and the r sum, so lanes 0..4 evaluate the five exponentials in one
    // call and lanes 0, 1 the two quotients in one division: the same functions on the same arguments (the
    // results are those of the serial chain bit for bit), a third of its instructions in sequence.
    const h1 rh = (h1)rr;
    const float pp_ = st.pp, aa_ = st.aa, bb_ = st.bb;
    const float ww = st.tf + k;
    const float p1 = (pp_ > ww) ? pp_ : ww;
    const float ww2 = st.td + pp_;
    const float p2 = (ww2 > k) ? ww2 : k;
    const float arg = lane == 0 ? pp_ - p1 : lane == 1 ? ww - p1 : lane == 2 ? ww2 - p2 : lane == 3 ? k - p2 : -(float)rh;
    const float e = expf(arg);
    auto lane_of = [](float x, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), l)); };
    const float e1 = lane_of(e, 0), e2 = lane_of(e, 1), e1n = lane_of(e, 2), e2n = lane_of(e, 3), es = lane_of(e, 4);
    const float num = lane == 0 ? (e1 * aa_ + e2 * v) : 1.0f;
    const float den = lane == 0 ? (e1 * bb_ + e2) : (1.0f + es);
    const float quo = num / den;
    const float wkv = lane_of(quo, 0), s32 = lane_of(quo, 1);  // s32 = 1 / (1 + exp(-r)): sigmoid_h_fast's value
    if (lane == 0) {
      const uint32_t frac = __float_as_uint(s32) & 0x1FFFu;
      const bool safe = s32 > 1e-4f && (frac < 0x1000u - 64u || frac > 0x1000u + 64u);
      const h1 r = safe ? (h1)s32 : sigmoid_h_exact(rh);
      a.rwkv_out[n] = r * (h1)wkv;
      a.aa_out[n] = e1n * aa_ + e2n * v;
      a.bb_out[n] = e1n * bb_ + e2n;
      a.pp_out[n] = p2;
    }
  };

  if constexpr (SINGLE) {
    // no load follows the rows: every wait for a chunk is exact
    if (c0 < c1) channel(c0, cur, st);
    return;
  }
  // Several channels per wave: the next channel's rows are requested ahead of the current one's
  // products where two sets of rows fit in the register file; long rows are loaded one channel
  // at a time.
  constexpr bool kAhead = U8 ? NCH <= 2 : NCH <= 5;
  for (int n = c0; n < c1; n++) {
    Rows3 nxt;
    Chan nst;
    if constexpr (kAhead)
      if (n + 1 < c1) {
        load_chan(nst, n + 1);
        load3(nxt, n + 1, true);
      }
    channel(n, cur, st);
    if (n + 1 < c1) {
      if constexpr (kAhead) {
        cur = nxt;
        st = nst;
      } else {
        load_chan(st, n + 1);
        load3(cur, n + 1, true);
      }
    }
  }
}

// ===========================================================================
// The general row-streaming kernel: up to four matrices ("segments") in one launch,
// each with its own staged activation vector and per-output epilogue.  Global row g
// belongs to the segment s with start[s] <= g < start[s+1].
// ===========================================================================
enum Prologue : int {
  P_COPY = 0,   // stage vec0 from global memory
  P_LN = 1,     // stage LN(x)
  P_LN_MIX = 2  // stage mix(LN(x), sx, mix[i]) for i < nvec; workgroup 0 writes LN(x) to xx_out
};

enum Epilogue : int {
  E_STORE_F16 = 0,  // out_h[n] = h(sum)
  E_STORE_F32 = 1,  // out_f[n] = sum
  E_RESIDUAL = 2,   // out_h[n] = x[n] + h(sum)                        att.cu:213-215
  E_SIGMOID = 3,    // out_h[n] = sigmoid(h(sum))                      ffn.cu:78-79
  E_RELU2 = 4,      // out_h[n] = relu(h(sum))^2                       ffn.cu:80-81
  E_FFN_OUT = 5,    // out_h[n] = fma(h(sum), r[n], x[n]) [/ 2]        ffn.cu:82-85, model_forward.cpp:173-175
  E_LOGITS = 6,     // out_f[n] = float(h(sum))                        model_forward.cpp:184-188
  E_SILU = 7        // out_h[n] = silu(h(sum))                         att.cu:289-290
};

struct Seg {
  WMat w;
  int vec;  // which staged vector this segment multiplies
  int epi;
  void* out;
};

struct RowsArgs {
  int K;          // length of every staged vector == K of every segment
  Split split;    // rows of all segments over the waves of the grid (set at launch)
  int nseg, nvec; // segments, staged vectors
  int prologue;
  int start[kMaxSeg + 1];  // first global row of each segment; start[nseg] = total rows (host bookkeeping)
  int bstart[kMaxSeg + 1]; // first batch of each segment for the launch's R (set at launch)
  Seg seg[kMaxSeg];
  // prologue inputs
  const h1* vec0;                      // P_COPY
  const h1 *x, *sx, *ln_w, *ln_b;      // P_LN, P_LN_MIX
  const h1* mix[kMaxSeg];              // P_LN_MIX
  h1* xx_out;                          // P_LN_MIX
  // epilogue inputs
  const h1* res_x;  // E_RESIDUAL, E_FFN_OUT
  const h1* res_r;  // E_FFN_OUT
  int res_n;        // elements of res_x / res_r that may be read (1 when no epilogue uses them)
  float* mirror;    // E_LOGITS: second destination of every value (memory the host reads), or null
  int div2;
#ifdef FRHIP_TIMELINE
  int tl_slot;  // where the launch leaves its timestamps
#endif
};

// Every workgroup serves one segment only: workgroups wg_start[s] .. wg_start[s+1]-1 serve segment s, whose batches are
// split over their waves by seg_split[s]; the workgroup then loads, stages and sums for that segment alone.  A second
// kernel argument of the launches of that form only: the arguments of the shared form stay as long as they were (56
// bytes of padding at their end, read by nobody, took 0.7-1.4 % off the decode rate of every model measured).
struct ExclArgs {
  int wg_start[kMaxSeg + 1];
  Split seg_split[kMaxSeg];
};
struct NoExclArgs {};

__device__ __forceinline__ void run_epilogue(const RowsArgs& a, const Seg& sg, int n, float sum, h1 ex, h1 er) {
  switch (sg.epi) {
    case E_STORE_F16: static_cast<h1*>(sg.out)[n] = (h1)sum; break;
    case E_STORE_F32: static_cast<float*>(sg.out)[n] = sum; break;
    case E_RESIDUAL: static_cast<h1*>(sg.out)[n] = ex + (h1)sum; break;
    case E_SIGMOID: static_cast<h1*>(sg.out)[n] = sigmoid_h((h1)sum); break;
    case E_RELU2: {
      h1 t = (h1)sum;
      static_cast<h1*>(sg.out)[n] = (t > (h1)0.0f) ? (t * t) : (h1)0.0f;
      break;
    }
    case E_FFN_OUT: {
      h1 o = __builtin_fmaf16((h1)sum, er, ex);  // __hfma: one rounding
      if (a.div2) o = o / (h1)2.0f;
      static_cast<h1*>(sg.out)[n] = o;
      break;
    }
    case E_LOGITS: {
      const float v = (float)(h1)sum;
      static_cast<float*>(sg.out)[n] = v;
      if (a.mirror) a.mirror[n] = v;
      break;
    }
    case E_SILU: static_cast<h1*>(sg.out)[n] = silu_h((h1)sum); break;
    default: break;
  }
}

// MULTI = a wave has several batches: two batches live in registers and alternate, the
// loads of one in flight while the other is consumed.
// PRO = the prologue, known at compile time so that its loads form straight-line code.
//
// Order of the global loads: operands of the prologue, then the first batch of rows with the
// per-row operands of its epilogue, all before the first wait and none inside a branch (threads
// and waves without work read a valid duplicate).  Vector loads return in the order they were
// issued, so the prologue runs while the rows are in flight and the products start on the
// first chunks that arrive; a load inside a branch would make the number of loads in flight
// path-dependent and turn every later wait into a wait for all of them.
// EXCL: every workgroup serves one segment only (RowsArgs::exclusive); a parameter of the kernel, not a field it tests,
// because the test and the lookups behind it cost every launch of the shared form 1.5-2 % (decode tok/s with and
// without the branch in the code: 1 428 against 1 449 binary16, 746 against 761 for the 3B RWKV-5.2).
template <int R, int NCH, bool U8, bool MULTI, int PRO, bool EXCL, class XA>
__device__ __forceinline__ void rows_body(const RowsArgs& a, const XA& xa) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[2 * kWaves];
  FR_TL_DECL;
  FR_TL(0);  // entry
  // One field from every 64-byte line of the kernel arguments is requested up front, so that the
  // scalar loads further down (issued where each field is first needed) hit the scalar cache.
  asm volatile("" ::"s"(a.K), "s"(a.seg[0].out), "s"(a.seg[1].out), "s"(a.seg[2].out), "s"(a.seg[3].out), "s"(a.vec0),
               "s"(a.res_x));
  static_assert(offsetof(RowsArgs, seg[0].out) / 64 == 1 && offsetof(RowsArgs, seg[1].out) / 64 == 2 &&
                    offsetof(RowsArgs, seg[2].out) / 64 == 3 && offsetof(RowsArgs, seg[3].out) / 64 == 4 &&
                    offsetof(RowsArgs, vec0) / 64 == 5 && offsetof(RowsArgs, mix[2]) / 64 == 5 &&
                    offsetof(RowsArgs, mix[3]) / 64 == 6 && offsetof(RowsArgs, res_x) / 64 == 6 &&
                    offsetof(RowsArgs, div2) / 64 == 6,
                "the list above must name one field of every 64-byte line of the arguments the shared form reads");
  if constexpr (EXCL) asm volatile("" ::"s"(xa.wg_start[1]), "s"(xa.seg_split[3].rem));
  const int K = a.K;
  const int nchunk = U8 ? (K >> 4) : (K >> 3);
  const size_t row_bytes = U8 ? (size_t)K : 2 * (size_t)K;
  // binary16: nvec staged activation vectors; uint8: one pre-scaled fp32 vector xr per segment
  constexpr int kPad = NCH * kWave;
  constexpr size_t kVecBytes = staged_bytes(NCH, U8);
  auto vec_at = [&](int i) { return smem + (size_t)i * kVecBytes; };
  __shared__ float qred[kWaves][kMaxSeg * kQSums];
  float qtv = 0.f;  // uint8: lane v holds total v of (Sx, Smy) x segments

  const int lane = threadIdx.x & (kWave - 1);
  // Work is dealt in batches of R rows that never straddle two matrices: segment s owns the batches
  // bstart[s] .. bstart[s+1]-1 (its last batch may be short), and the batches of all segments are
  // split evenly over the waves of the grid.  One batch therefore multiplies one staged vector.
  // The wave index is made visibly uniform: otherwise the lookups in the kernel arguments
  // (segment table, row addresses) become vector loads that every weight load has to wait for.
  int g0, g1;
  int ws = 0;  // exclusive launches: the one segment this workgroup serves
  if constexpr (EXCL) {
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++) ws += (i < a.nseg && (int)blockIdx.x >= xa.wg_start[i]) ? 1 : 0;
    const int wgs = xa.wg_start[ws + 1] - xa.wg_start[ws], lb = (int)blockIdx.x - xa.wg_start[ws];
    const Split sp = xa.seg_split[ws];
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // numbered as grid_wave numbers them, within the segment's workgroups
    split_even(sp, sp.rem != 0 ? wv * wgs + lb : lb * kWaves + wv, g0, g1);
    g0 += a.bstart[ws];
    g1 += a.bstart[ws];
  } else {
    split_even(a.split, grid_wave(a.split), g0, g1);
  }
  // does this workgroup need segment i's operands / staged vector j?
  auto serves_seg = [&](int i) { return EXCL ? i == ws : i < a.nseg; };
  auto serves_vec = [&](int j) { return EXCL ? j == a.seg[ws].vec : j < a.nvec; };
  const int qmul = EXCL ? 0 : 1;  // exclusive: the segment's Sx, Smy are totals 0, 1; else segment s has 2 s, 2 s + 1

  struct Meta {
    int seg, loc0, nvalid;  // segment, first row within it, rows of the batch that exist
    // Per-row operands of the epilogue, lane r holding those of row r.  They are requested with the
    // batch's weights: asked for after the products they would cost a whole memory latency at the
    // end of the launch.
    h1 ex, er, qrx, qmx;
  };
  // Row addresses and extents of a batch; `live` = the batch is this wave's to finish.
  struct Where {
    const void* rows[R];
    int nbytes[R];
  };
  auto locate = [&](Meta& m, Where& wh, int bi, bool live) {
    int sg = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++) sg += (i < a.nseg && bi >= a.bstart[i]) ? 1 : 0;
    const int n = a.seg[sg].w.N;
    m.seg = sg;
    m.loc0 = (bi - a.bstart[sg]) * R;
    m.nvalid = n - m.loc0 < R ? n - m.loc0 : R;
    if (!live) m.nvalid = 0;
    const unsigned char* base = a.seg[sg].w.data;
#pragma unroll
    for (int r = 0; r < R; r++) {
      const bool have = live && m.loc0 + r < n;  // surplus slots and idle waves read nothing
      wh.rows[r] = base + (size_t)(have ? m.loc0 + r : 0) * row_bytes;
      wh.nbytes[r] = have ? (int)row_bytes : 0;
    }
  };
  // issue the loads of a located batch: its rows (chunks J0 .. J1-1), then the per-row operands of
  // its epilogue
  auto request_rows = [&](RowBatch<R, NCH, U8>& b, const Where& wh, auto j0, auto j1) {
    b.template load<decltype(j0)::value, decltype(j1)::value>(wh.rows, wh.nbytes, lane);
  };
  auto request_ops = [&](Meta& m) {
    const int n = a.seg[m.seg].w.N;
    const int nl = m.loc0 + lane < n ? m.loc0 + lane : n - 1;
    m.ex = m.er = (h1)0.0f;
    if constexpr (PRO == P_COPY) {  // the launches with residual epilogues all stage a ready vector
      const int ri = nl < a.res_n ? nl : a.res_n - 1;
      m.ex = a.res_x[ri];
      m.er = a.res_r[ri];
    }
    if constexpr (U8) {
      m.qrx = a.seg[m.seg].w.rx[nl];
      m.qmx = a.seg[m.seg].w.mx[nl];
    }
  };
  using J0 = std::integral_constant<int, 0>;
  // (a wave with several batches streams anyway: its first batch goes out whole)
  using JH = std::integral_constant<int, MULTI ? NCH : RowBatch<R, NCH, U8>::kHead>;
  using JN = std::integral_constant<int, NCH>;
  auto fetch = [&](RowBatch<R, NCH, U8>& b, Meta& m, int bi, bool live) {
    Where wh;
    locate(m, wh, bi, live);
    request_rows(b, wh, J0{}, JN{});
    request_ops(m);
  };
  auto consume = [&](const RowBatch<R, NCH, U8>& b, const Meta& m) {
    const Seg& sg = a.seg[m.seg];
    float acc[R];
    b.dot_shared(vec_at(U8 ? m.seg : sg.vec), lane, acc);
    FR_TL_AFTER(8, acc[0]);  // products done (of the wave's last batch)
    float mine = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
      const float t = wave_sum(acc[r]);
      if (lane == r) mine = t;
    }
    FR_TL_AFTER(9, mine);  // reduced
    if (lane < m.nvalid) {
      const int n = m.loc0 + lane;
      if constexpr (U8) {
        // lane v of qtv holds total v of (Sx, Smy) x segments; the segment is uniform here
        const float sx_ = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qtv), m.seg * kQSums * qmul + 0));
        const float smy_ = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qtv), m.seg * kQSums * qmul + 1));
        mine = finish_q(mine, (float)m.qrx, (float)m.qmx, sx_, smy_);
      }
      run_epilogue(a, sg, n, mine, m.ex, m.er);
    }
  };

  // where the first batch lives: scalar work, done before any load is requested
  Meta mA;
  Where whA;
  locate(mA, whA, g0 < g1 ? g0 : a.bstart[a.nseg] - 1, g0 < g1);

  // ---- operands of the prologue ----
  // P_COPY: the vector (one segment; uint8: with its ry, my) in passes of one 8-element group per
  // thread; P_LN / P_LN_MIX: K <= 8 * kThreads, one group per thread.  Only threads that own a
  // group load (every byte requested here passes through the compute unit's vector memory
  // pipeline ahead of the rows): branches are harmless before the rows, whose count is fixed.
  // P_COPY, uint8 (three operand vectors: the vector, ry, my): the first four waves of the workgroup (one per SIMD, the
  // ones the compute unit serves first) load and stage all of them, so the pieces are at the head of the compute unit's
  // queue (data returns in request order across the waves: an operand requested by wave 7 behind the rows of waves 0-6
  // arrives after them).  Where a batch is more than 8 loads the rows of those four waves alone fill what a compute unit
  // keeps in flight (about 64 KB) and the other four would be held at their load instructions, and with them the barrier
  // that releases the staged vector: there they go to the barrier first and request their rows behind it.
  // Measured (decode tok/s, one box, alternating): RWKV-4 1.5B uint8 1 634 -> 1 644, RWKV-5.2 3B uint8 845 -> 851; the same
  // for binary16 (one operand vector) 1 430 -> 1 424 and 746 -> 740, so binary16 keeps every thread loading its own group.
  constexpr bool kStagerMode = PRO == P_COPY && U8;
  constexpr int kStageWaves = kStagerMode ? 4 : kWaves, kStageThreads = kStageWaves * kWave;
  constexpr int kCopyPasses = (NCH * kWave * (U8 ? 2 : 1) + kStageThreads - 1) / kStageThreads;
  const bool stager = (int)threadIdx.x < kStageThreads;  // uniform within a wave
  const int ngrp = K >> 3;
  const bool own = (int)threadIdx.x < ngrp;
  const int e0 = threadIdx.x * 8;
  h8 cx[kCopyPasses] = {}, cry[kCopyPasses] = {}, cmy[kCopyPasses] = {};
  h8 xv{}, lg{}, lb{}, sxv{}, mixv[kMaxSeg] = {}, qry[kMaxSeg] = {}, qmy[kMaxSeg] = {};
  if constexpr (PRO == P_COPY) {
    if (stager) {
#pragma unroll
      for (int p = 0; p < kCopyPasses; p++) {
        const int g = (int)threadIdx.x + p * kStageThreads;
        if (g < ngrp) {
          cx[p] = reinterpret_cast<const h8*>(a.vec0)[g];
          if constexpr (U8) {
            cry[p] = reinterpret_cast<const h8*>(a.seg[0].w.ry)[g];
            cmy[p] = reinterpret_cast<const h8*>(a.seg[0].w.my)[g];
          }
        }
      }
    }
  } else if (own) {
    xv = *reinterpret_cast<const h8*>(a.x + e0);
    lg = *reinterpret_cast<const h8*>(a.ln_w + e0);
    lb = *reinterpret_cast<const h8*>(a.ln_b + e0);
    if constexpr (PRO == P_LN_MIX) {
      sxv = *reinterpret_cast<const h8*>(a.sx + e0);
#pragma unroll
      for (int i = 0; i < kMaxSeg; i++)
        if (serves_vec(i)) mixv[i] = *reinterpret_cast<const h8*>(a.mix[i] + e0);
    }
    if constexpr (U8) {
#pragma unroll
      for (int i = 0; i < kMaxSeg; i++)
        if (serves_seg(i)) {
          qry[i] = *reinterpret_cast<const h8*>(a.seg[i].w.ry + e0);
          qmy[i] = *reinterpret_cast<const h8*>(a.seg[i].w.my + e0);
        }
    }
  }

  FR_TL(1);  // the prologue's operands requested
  // ---- first batch of rows: the chunks that go out ahead of the prologue (see RowBatch::kHead) ----
  RowBatch<R, NCH, U8> A;
  constexpr bool kAllRowsFirst = R * NCH <= 8;
  if constexpr (kStagerMode) {
    if (kAllRowsFirst || stager) {
      request_rows(A, whA, J0{}, JN{});
      request_ops(mA);
    }
  } else {
    request_rows(A, whA, J0{}, JH{});
    if constexpr (!U8) request_ops(mA);
  }
  FR_TL(2);  // first rows requested

  // ---- prologue: stage the activation vector(s) in LDS ----
  // uint8: Sx and Smy of every staged vector are needed only when a row is finished.  They are summed behind the
  // barrier that releases the staged vectors and behind the last row requests (below), from the values each thread
  // keeps in `qx`, while the rows are on their way.
  float part[kMaxSeg * kQSums];
#pragma unroll
  for (int i = 0; i < kMaxSeg * kQSums; i++) part[i] = 0.f;
  h8 qx[kMaxSeg] = {};
  {
    if constexpr (PRO == P_COPY) {
      if (stager) {
#pragma unroll
        for (int p = 0; p < kCopyPasses; p++) {
          const int g = (int)threadIdx.x + p * kStageThreads;
          if (g < ngrp) {
            if constexpr (!U8)
              reinterpret_cast<h8*>(vec_at(0))[g] = cx[p];
            else
              stage_q(reinterpret_cast<float*>(vec_at(0)), g, kPad, cx[p], cry[p], cmy[p], part);
          }
        }
      }
    } else if (PRO == P_LN && K > kFusedMaxC) {
      // a vector wider than one group per thread (the head of a model with n_embd > 4096): the same
      // normalisation with every thread looping over its groups; x is re-read from the cache
      const h8* xp8 = reinterpret_cast<const h8*>(a.x);
      float s1 = 0.f;
      for (int g = threadIdx.x; g < ngrp; g += kThreads) {
        const h8 x = xp8[g];
#pragma unroll
        for (int i = 0; i < 8; i++) s1 += (float)x[i];
      }
      const float mean = block_sum1<kWaves>(s1, red) / (float)K;
      float s2 = 0.f;
      for (int g = threadIdx.x; g < ngrp; g += kThreads) {
        const h8 x = xp8[g];
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const float d = (float)x[i] - mean;
          s2 += d * d;
        }
      }
      float var = block_sum1<kWaves>(s2, red + kWaves) / (float)K;
      var = var > 0.f ? var : 0.f;
      const float inv = 1.0f / sqrtf(var + 1e-5f);
      for (int g = threadIdx.x; g < ngrp; g += kThreads) {
        const h8 x = xp8[g], gm = reinterpret_cast<const h8*>(a.ln_w)[g], bt = reinterpret_cast<const h8*>(a.ln_b)[g];
        h8 xx;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          const h1 n = (h1)(((float)x[i] - mean) * inv);
          xx[i] = (n * gm[i]) + bt[i];
        }
        if constexpr (!U8) {
          reinterpret_cast<h8*>(vec_at(0))[g] = xx;
        } else {
          const h8 ry = reinterpret_cast<const h8*>(a.seg[0].w.ry)[g], my = reinterpret_cast<const h8*>(a.seg[0].w.my)[g];
          stage_q(reinterpret_cast<float*>(vec_at(0)), g, kPad, xx, ry, my, part);
        }
      }
    } else {
      LnOut ln = ln_regs(xv, lg, lb, own, K, red);
      FR_TL_AFTER(3, (float)ln.xx[0]);  // normalised (the vector has arrived, both reductions are through)
      if (ln.active) {
        if constexpr (!U8) {
          if constexpr (PRO == P_LN) {
            reinterpret_cast<h8*>(vec_at(0))[threadIdx.x] = ln.xx;
          } else {
#pragma unroll
            for (int i = 0; i < kMaxSeg; i++)
              if (serves_vec(i)) reinterpret_cast<h8*>(vec_at(i))[threadIdx.x] = mix8(ln.xx, sxv, mixv[i]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < kMaxSeg; i++) {
            if (serves_seg(i)) {
              h8 x = ln.xx;
              if constexpr (PRO == P_LN_MIX) {
                // segment i multiplies staged vector seg[i].vec; pick its mix without dynamic register indexing
                h8 mx8 = mixv[0];
#pragma unroll
                for (int j = 1; j < kMaxSeg; j++)
                  if (a.seg[i].vec == j) mx8 = mixv[j];
                x = mix8(ln.xx, sxv, mx8);
              }
              stage_xr(reinterpret_cast<float*>(vec_at(i)), threadIdx.x, kPad, x, qry[i]);
              qx[i] = x;
            }
          }
        }
        if (PRO == P_LN_MIX && blockIdx.x == 0) *reinterpret_cast<h8*>(a.xx_out + e0) = ln.xx;
      }
    }
    for (int i = 0; i < (U8 ? a.nseg : a.nvec); i++)
      if (U8 ? serves_seg(i) : serves_vec(i)) zero_pad<U8>(vec_at(i), nchunk, kPad);
    // (a ready vector is staged within a fraction of a microsecond and its rows are few: there the sums stay ahead of the barrier)
    if constexpr (U8 && PRO == P_COPY) publish_qsums(part, a.nseg * kQSums, qred);  // (one segment: never exclusive)
    FR_TL(4);  // staged: at the barrier
    __syncthreads();
    FR_TL(5);  // through the barrier
  }
  // ---- the rest of the first batch ----
  if constexpr (kStagerMode) {
    if (!kAllRowsFirst && !stager) {
      request_rows(A, whA, J0{}, JN{});
      request_ops(mA);
    }
  } else {
    request_rows(A, whA, JH{}, JN{});
    // uint8: the per-row operands (two more 2-byte loads per lane: rx, mx) go out behind all rows of the batch; ahead of
    // the prologue they cost these launches more than the memory latency they save at the end (decode kernels 0.588 ->
    // 0.583 ms per token; binary16, with at most two such loads, the other way round: 0.662 -> 0.669).
    if constexpr (U8) request_ops(mA);
  }
  if constexpr (U8) {
    // (every thread reaches the second barrier; threads without a group add zeros; the wide layernorm has summed already)
    if constexpr (PRO != P_COPY) {
#pragma unroll
      for (int i = 0; i < kMaxSeg; i++)
        if (serves_seg(i)) {
          if (EXCL)
            sum_q(qx[i], qmy[i], part);
          else
            sum_q(qx[i], qmy[i], part + i * kQSums);
        }
      publish_qsums(part, (EXCL ? 1 : a.nseg) * kQSums, qred);
      __syncthreads();
    }
    qtv = gather_qsums((EXCL ? 1 : a.nseg) * kQSums, qred);
  }
  FR_TL_AFTER(6, qtv);  // all rows of the first batch requested (uint8: Sx, Smy gathered)

  if constexpr (!MULTI) {
    consume(A, mA);  // the host guarantees at most one batch per wave
  } else {
    // Two register sets alternate.  Each "fetch the next, consume the current" pair is straight-line
    // code, so the loads of the next batch stay in flight while the current one is consumed.
    RowBatch<R, NCH, U8> B;
    Meta mB;
    int g = g0;
    if (g < g1) {
      for (;;) {
        if (g + 1 >= g1) {
          consume(A, mA);
          break;
        }
        fetch(B, mB, g + 1, true);
        consume(A, mA);
        g += 1;
        if (g + 1 >= g1) {
          consume(B, mB);
          break;
        }
        fetch(A, mA, g + 1, true);
        consume(B, mB);
        g += 1;
      }
    }
  }
  FR_TL(10);  // epilogue issued
  FR_TL_FLUSH(a.tl_slot);  // waits for the wave's stores, notes the time, writes the notes
}

template <int R, int NCH, bool U8, bool MULTI, int PRO>
__global__ __launch_bounds__(kThreads) void rows_kernel(RowsArgs a) {
  rows_body<R, NCH, U8, MULTI, PRO, false>(a, NoExclArgs{});
}

// The form in which every workgroup serves one segment (layernorm + mix launches of several matrices only).
template <int R, int NCH, bool U8, bool MULTI>
__global__ __launch_bounds__(kThreads) void rows_excl_kernel(RowsArgs a, ExclArgs xa) {
  rows_body<R, NCH, U8, MULTI, P_LN_MIX, true>(a, xa);
}

// ===========================================================================
// Layernorm of one token's vector and its token-shift mixes as a kernel of its own, for models
// wider than the fused prologues take (n_embd > 4096): out[i] = mix(LN(x), sx, mix[i]) for
// i < nmix, xx_out = LN(x)   (kernels/cuda/layer_norm.cu:60-69, att.cu:90-113).
// One workgroup; thread t owns the 8-element groups t, t + 512, ... (at most four: n_embd <= 16384).
// ===========================================================================
struct LnMixOne {
  int C, nmix;
  const h1 *x, *sx, *ln_w, *ln_b;
  const h1* mix[4];
  h1* out[4];
  h1* xx_out;
};

__global__ __launch_bounds__(kThreads) void ln_mix_one_kernel(LnMixOne a) {
  constexpr int G = kMaxC / (8 * kThreads);
  __shared__ float red[2 * kWaves];
  const int ngrp = a.C >> 3;
  h8 xv[G], gm[G], bt[G], sx[G];
  bool own[G];
#pragma unroll
  for (int i = 0; i < G; i++) {
    const int g = threadIdx.x + i * kThreads;
    own[i] = g < ngrp;
    const int gc = own[i] ? g : 0;
    xv[i] = reinterpret_cast<const h8*>(a.x)[gc];
    gm[i] = reinterpret_cast<const h8*>(a.ln_w)[gc];
    bt[i] = reinterpret_cast<const h8*>(a.ln_b)[gc];
    sx[i] = reinterpret_cast<const h8*>(a.sx)[gc];
  }
  float s1 = 0.f;
#pragma unroll
  for (int i = 0; i < G; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) s1 += own[i] ? (float)xv[i][e] : 0.f;
  const float mean = block_sum1<kWaves>(s1, red) / (float)a.C;
  float s2 = 0.f;
#pragma unroll
  for (int i = 0; i < G; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float d = (float)xv[i][e] - mean;
      s2 += own[i] ? d * d : 0.f;
    }
  float var = block_sum1<kWaves>(s2, red + kWaves) / (float)a.C;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
#pragma unroll
  for (int i = 0; i < G; i++) {
    if (!own[i]) continue;
    const int g = threadIdx.x + i * kThreads;
    h8 xx;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const h1 n = (h1)(((float)xv[i][e] - mean) * inv);
      xx[e] = (n * gm[i][e]) + bt[i][e];
    }
    reinterpret_cast<h8*>(a.xx_out)[g] = xx;
    for (int m = 0; m < a.nmix; m++)
      reinterpret_cast<h8*>(a.out[m])[g] = mix8(xx, sx[i], reinterpret_cast<const h8*>(a.mix[m])[g]);
  }
}

// ===========================================================================
// WKV-4 update of one token as a kernel of its own (kernels/cuda/att.cu:30-62), one thread per
// channel: the arithmetic of att_front_v4_kernel's last step, for models wider than that
// kernel takes.  r has already passed through the sigmoid.
// ===========================================================================
struct Wkv4One {
  int C;
  const float *k, *v, *aa, *bb, *pp, *td, *tf;
  const h1* r;
  h1* rwkv_out;
  float *aa_out, *bb_out, *pp_out;
};

__global__ __launch_bounds__(256) void wkv4_one_kernel(Wkv4One a) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= a.C) return;
  const float k = a.k[n], v = a.v[n];
  const h1 r = a.r[n];
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

// ===========================================================================
// Rows longer than the largest register tiling (K > 9216 binary16 / 16384 uint8 elements: the
// ffn value matrix of the 3B and larger models).  One matrix against one ready vector (P_COPY).
// A workgroup owns consecutive rows; a row is cut into `nslice` slices of `cs` chunks per lane
// (cs <= NCH), and the (row, slice) items of the workgroup are dealt evenly to its eight waves,
// so that the waves stay balanced also where the matrix has fewer rows than the grid has waves.
// A wave streams its items through two alternating register sets and leaves one partial sum
// per item in LDS; after a barrier one thread per row adds the row's partials in slice order
// (a fixed order: results do not depend on timing) and runs the epilogue.
// The whole vector is staged in LDS (2 K bytes; uint8: 4 K bytes of x * ry in fp32).
// ===========================================================================
struct SliceGeom {
  int nslice, cs;    // slices per row, chunks per lane and slice
  int padchunks;     // chunks of the staged vector, padding included: (nslice - 1) * cs * 64 + NCH * 64
  Split rows;        // rows over the workgroups of the grid
  int part_offset;   // byte offset of the partial sums in dynamic LDS
};

template <int NCH, bool U8>
__global__ __launch_bounds__(kThreads) void rows_sliced_kernel(RowsArgs a, SliceGeom g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float qred[kWaves][kMaxSeg * kQSums];
  const int K = a.K;
  const int nchunk = U8 ? (K >> 4) : (K >> 3);
  const int row_bytes = U8 ? K : 2 * K;
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const Seg& sg = a.seg[0];
  float* partials = reinterpret_cast<float*>(smem + g.part_offset);
  int r0, r1;  // this workgroup's rows
  split_even(g.rows, blockIdx.x, r0, r1);
  const int nrows = r1 - r0;
  const int items = nrows * g.nslice;
  const int i0 = (int)(((long)items * wv) / kWaves), i1 = (int)(((long)items * (wv + 1)) / kWaves);

  // per-row operands of the epilogue, thread t holding those of row r0 + t (first pass of the final loop)
  h1 ex = (h1)0.0f, er = (h1)0.0f, qrx = (h1)0.0f, qmx = (h1)0.0f;
  if ((int)threadIdx.x < nrows) {
    const int n = r0 + threadIdx.x;
    const int ri = n < a.res_n ? n : a.res_n - 1;
    ex = a.res_x[ri];
    er = a.res_r[ri];
    if constexpr (U8) {
      qrx = sg.w.rx[n];
      qmx = sg.w.mx[n];
    }
  }

  // item -> (row, slice); the slice's extent ends where the slice does
  auto fetch = [&](RowBatch<1, NCH, U8>& b, int row, int sl, bool live) {
    const void* rows[1] = {sg.w.data + (size_t)(live ? row : 0) * (size_t)row_bytes};
    const int end = (sl + 1) * g.cs * (kWave * 16);
    const int nbytes[1] = {live ? (end < row_bytes ? end : row_bytes) : 0};
    b.load_slice(rows, nbytes, lane, sl * g.cs * (kWave * 16));
  };

  RowBatch<1, NCH, U8> A, B;
  int row = r0 + i0 / g.nslice, sl = i0 % g.nslice;
  fetch(A, row, sl, i0 < i1);

  // ---- the vector, staged under the first loads ----
  float part[kQSums] = {0.f, 0.f};
  for (int gi = threadIdx.x; gi < (K >> 3); gi += kThreads) {
    const h8 x = reinterpret_cast<const h8*>(a.vec0)[gi];
    if constexpr (!U8) {
      reinterpret_cast<h8*>(smem)[gi] = x;
    } else {
      const h8 ry = reinterpret_cast<const h8*>(sg.w.ry)[gi];
      const h8 my = reinterpret_cast<const h8*>(sg.w.my)[gi];
      stage_q(reinterpret_cast<float*>(smem), gi, g.padchunks, x, ry, my, part);
    }
  }
  zero_pad<U8>(smem, nchunk, g.padchunks);
  if constexpr (U8) publish_qsums(part, kQSums, qred);
  __syncthreads();
  float qtv = 0.f;
  if constexpr (U8) qtv = gather_qsums(kQSums, qred);

  auto consume = [&](const RowBatch<1, NCH, U8>& b, int row_, int sl_) {
    float acc[1] = {0.f};
    b.dot_add(smem, lane, sl_ * g.cs * kWave, g.padchunks, acc);
    const float t = wave_sum(acc[0]);
    if (lane == 0) partials[(row_ - r0) * g.nslice + sl_] = t;
  };
  auto advance = [&](int& r_, int& s_) {
    s_ += 1;
    if (s_ == g.nslice) {
      s_ = 0;
      r_ += 1;
    }
  };
  // fetch the next item, consume the current one; the two register sets alternate
  for (int i = i0; i < i1;) {
    int nrow = row, nsl = sl;
    advance(nrow, nsl);
    if (i + 1 >= i1) {
      consume(A, row, sl);
      break;
    }
    fetch(B, nrow, nsl, true);
    consume(A, row, sl);
    row = nrow;
    sl = nsl;
    i += 1;
    advance(nrow, nsl);
    if (i + 1 >= i1) {
      consume(B, row, sl);
      break;
    }
    fetch(A, nrow, nsl, true);
    consume(B, row, sl);
    row = nrow;
    sl = nsl;
    i += 1;
  }
  __syncthreads();

  // ---- one thread per row: partials in slice order, then the epilogue ----
  for (int t = threadIdx.x; t < nrows; t += kThreads) {
    const int n = r0 + t;
    if (t >= kThreads) {  // more rows than threads: operands of the later passes
      const int ri = n < a.res_n ? n : a.res_n - 1;
      ex = a.res_x[ri];
      er = a.res_r[ri];
      if constexpr (U8) {
        qrx = sg.w.rx[n];
        qmx = sg.w.mx[n];
      }
    }
    float sum = 0.f;
    for (int s_ = 0; s_ < g.nslice; s_++) sum += partials[t * g.nslice + s_];
    if constexpr (U8) {
      const float q0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qtv), 0));
      const float q1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(qtv), 1));
      sum = finish_q(sum, (float)qrx, (float)qmx, q0, q1);
    }
    run_epilogue(a, sg, n, sum, ex, er);
  }
}

// ===========================================================================
// RWKV-5.1/5.2 one-token state update, per head (kernels/cuda/att.cu:64-81,296-329):
//   a_ij = k_i v_j ; tmp_ij = u_i a_ij + s_ij ; out_j = sum_i r_i tmp_ij ; s_ij <- w_i s_ij + a_ij
// with the products and sums of tmp and s rounded separately (the reference uses
// __fmul_rn/__fadd_rn there), then groupnorm over the head's S outputs (fp32, eps 1e-5),
// rounding to half and the gate multiply in half.
// One workgroup of 256 threads per head: thread t owns value index j = t % 64 and the
// key rows i = (t / 64) * 16 ... +15; the four partial sums of out_j meet in LDS.
// S must be 64.
// ===========================================================================
struct Wkv5One {
  int H;
  int uw_head;  // 0: u, w are [H][S] (RWKV-5.1/5.2); 1: one value per head (RWKV-5.0)
  const float *s, *r, *k, *v, *w, *u, *lx_w, *lx_b;
  const h1* g;  // gate, or null (RWKV-5.0 has none)
  float* s_out;
  h1* gated_out;
};

__global__ __launch_bounds__(256) void wkv5_one_kernel(Wkv5One a) {
  constexpr int S = 64;
  __shared__ float rk[3][S];      // r, k, v of this head
  __shared__ float uw[2][S];      // u, w
  __shared__ float part[4][S];
  const int h = blockIdx.x, t = threadIdx.x;
  const int j = t & 63, ig = t >> 6;
  if (t < S) {
    rk[0][t] = a.r[h * S + t];
    rk[1][t] = a.k[h * S + t];
    rk[2][t] = a.v[h * S + t];
    uw[0][t] = a.u[a.uw_head ? h : h * S + t];
    uw[1][t] = a.w[a.uw_head ? h : h * S + t];
  }
  const float* sh = a.s + (size_t)h * S * S;
  float* so = a.s_out + (size_t)h * S * S;
  float sreg[16];
#pragma unroll
  for (int ii = 0; ii < 16; ii++) sreg[ii] = sh[(ig * 16 + ii) * S + j];
  __syncthreads();
  const float vj = rk[2][j];
  float acc = 0.f;
#pragma unroll
  for (int ii = 0; ii < 16; ii++) {
    const int i = ig * 16 + ii;
    const float aij = rk[1][i] * vj;
    const float ua = uw[0][i] * aij;
    const float tmp = ua + sreg[ii];
    const float ws = uw[1][i] * sreg[ii];
    so[i * S + j] = ws + aij;
    acc += rk[0][i] * tmp;
  }
  part[ig][j] = acc;
  __syncthreads();
  if (t < S) {
    const float o = ((part[0][t] + part[1][t]) + part[2][t]) + part[3][t];
    const float mean = wave_sum(o) / (float)S;
    const float d = o - mean;
    float var = wave_sum(d * d) / (float)S;
    var = var > 0.f ? var : 0.f;
    const float inv = 1.0f / sqrtf(var + 1e-5f);
    const int c = h * S + t;
    const float y = d * inv * a.lx_w[c] + a.lx_b[c];
    a.gated_out[c] = a.g ? (h1)y * a.g[c] : (h1)y;
  }
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

#define FR_TRY(expr)        \
  do {                      \
    int _e = (expr);        \
    if (_e != 0) return _e; \
  } while (0)

// The fused one-token kernels hold the activation vector as one 8-element group per thread; wider
// models run the same arithmetic as separate launches (layernorm + mixes, one product per matrix,
// state update), which costs them a few launches per layer where a launch moves 50 MB and more.
static int check_embd(int C) {
  if (C <= 0 || C % 16 != 0 || C > kMaxC)
    return set_error(FRHIP_ESHAPE, "n_embd must be a multiple of 16 and at most 16384");
  return 0;
}

static int check_lds(size_t bytes) {
  if (bytes > 64 * 1024) return set_error(FRHIP_ESHAPE, "vector operands exceed 64 KB of LDS");
  return 0;
}

// Chunks (16 bytes per lane) a lane holds per row.
static int chunks_per_lane(int K, bool u8) {
  const int nchunk = u8 ? K / 16 : K / 8;
  return (nchunk + kWave - 1) / kWave;
}

// Supported register tilings.  NCH is rounded up to one of these; R is then chosen so
// that a wave's rows fit in one batch when that needs at most kMaxLoads loads per lane.
static const int kNchSet[] = {1, 2, 3, 4, 5, 8, 9, 16, 18};
constexpr int kMaxLoads = 32;

static int round_nch(int nch) {
  for (int v : kNchSet)
    if (nch <= v) return v;
  return -1;
}

// Rows in flight per wave.  When all rows of a wave fit in kMaxLoads loads per lane they
// form one batch (multi = false); otherwise batches of at most kMaxLoads/2 loads alternate
// between two register sets.
static int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  return (e && atoi(e) > 0) ? atoi(e) : dflt;
}

// Batches of R rows that never straddle two segments: their number for a given R.
static long count_batches(const RowsArgs& a, int R) {
  long nb = 0;
  for (int s = 0; s < a.nseg; s++) nb += (a.seg[s].w.N + R - 1) / R;
  return nb;
}

// Workgroups per segment for a launch whose workgroups serve one segment each: in proportion to the segments'
// batches, at least one each, summing to the grid.  Returns false when the grid has fewer workgroups than segments.
static bool share_workgroups(const RowsArgs& a, int R, int grid, int (&wgs)[kMaxSeg]) {
  if (grid < a.nseg) return false;
  long nb[kMaxSeg], total = 0;
  for (int s = 0; s < a.nseg; s++) {
    nb[s] = (a.seg[s].w.N + R - 1) / R;
    total += nb[s];
  }
  int given = 0, widest = 0;
  for (int s = 0; s < a.nseg; s++) {
    wgs[s] = (int)((nb[s] * grid + total / 2) / total);
    if (wgs[s] < 1) wgs[s] = 1;
    given += wgs[s];
    if (nb[s] > nb[widest]) widest = s;
  }
  wgs[widest] += grid - given;  // rounding: the segment with the most batches takes the difference
  return wgs[widest] >= 1;
}

// Every segment's batches fit one per wave of its own workgroups?
static bool exclusive_fits(const RowsArgs& a, int R, int grid) {
  int wgs[kMaxSeg];
  if (!share_workgroups(a, R, grid, wgs)) return false;
  for (int s = 0; s < a.nseg; s++)
    if ((long)(a.seg[s].w.N + R - 1) / R > (long)wgs[s] * kWaves) return false;
  return true;
}

// A launch of several matrices after a layernorm can give every workgroup one matrix only: the workgroup then loads and
// stages one mixed vector (uint8: one set of ry / my, two sums) instead of all of them, at the price of a longer search
// for its place in the launch.  It pays from about 14 KB of operands saved per workgroup -- (nseg - 1) x (uint8: mix, ry,
// my; binary16: mix) x 2 K bytes.  Decode tok/s against the shared form on one box: RWKV-5.2 3B uint8 (K = 2560, four
// and two matrices: 46 and 15 KB) 809 -> 876; its four-matrix binary16 launch (15 KB) 747 -> 760; RWKV-4 1.5B uint8
// (K = 2048, two matrices: 12 KB) 1 666 -> 1 656 and binary16 (4 KB) 1 426 -> 1 419, which therefore stay shared.
// FRHIP_SEG_EXCLUSIVE=0 / 1 forces it off / on for every such launch.
static bool want_exclusive(const RowsArgs& a, bool u8) {
  static const int forced = getenv("FRHIP_SEG_EXCLUSIVE") ? atoi(getenv("FRHIP_SEG_EXCLUSIVE")) : -1;
  if (a.nseg < 2 || a.prologue != P_LN_MIX || forced == 0) return false;
  return forced > 0 || (long)(a.nseg - 1) * (u8 ? 3 : 1) * 2 * a.K >= 14 * 1024;
}

static int pick_r(const RowsArgs& a, int grid, int nch, bool u8, bool* multi) {
  static const int max_u8 = env_int("FRHIP_MAXLOADS_U8", kMaxLoads);
  const int kMaxLoads = u8 ? max_u8 : frhip::kMaxLoads;
  const long waves = (long)grid * kWaves;
  int rmax = kMaxLoads / nch;
  if (rmax < 1) rmax = 1;
  if (rmax > 6) rmax = 6;
  // the smallest R for which every wave gets at most one batch: a single register-resident batch
  for (int r = 1; r <= rmax; r++)
    if (want_exclusive(a, u8) ? exclusive_fits(a, r, grid) : count_batches(a, r) <= waves) {
      *multi = false;
      return r;
    }
  *multi = true;
  int r = (kMaxLoads / 2) / nch;
  if (r < 1) r = 1;
  // uint8 rows are half as long in bytes: eight of them per batch keep as many bytes in flight
  if (u8 && r >= 8) return 8;
  if (r > 4) r = 4;
  return r;
}

// false when the (R, NCH, MULTI) tiling is not compiled (pick_r never asks for one that is not)
template <int R, int NCH, bool U8, bool MULTI>
static void launch_rows_pro(int grid, size_t lds, hipStream_t st, const RowsArgs& a, const ExclArgs* xa) {
  switch (a.prologue) {
    case P_COPY: hipLaunchKernelGGL((rows_kernel<R, NCH, U8, MULTI, P_COPY>), dim3(grid), dim3(kThreads), lds, st, a); break;
    case P_LN: hipLaunchKernelGGL((rows_kernel<R, NCH, U8, MULTI, P_LN>), dim3(grid), dim3(kThreads), lds, st, a); break;
    default:
      if (xa)
        hipLaunchKernelGGL((rows_excl_kernel<R, NCH, U8, MULTI>), dim3(grid), dim3(kThreads), lds, st, a, *xa);
      else
        hipLaunchKernelGGL((rows_kernel<R, NCH, U8, MULTI, P_LN_MIX>), dim3(grid), dim3(kThreads), lds, st, a);
      break;
  }
}

template <int R, int NCH>
static bool launch_rows_rn(bool u8, bool multi, int grid, size_t lds, hipStream_t st, const RowsArgs& a, const ExclArgs* xa) {
  if (!multi) {
    if constexpr ((R * NCH <= kMaxLoads && R <= 6) || R == 1) {
      if (u8)
        launch_rows_pro<R, NCH, true, false>(grid, lds, st, a, xa);
      else
        launch_rows_pro<R, NCH, false, false>(grid, lds, st, a, xa);
      return true;
    }
  } else {
    if constexpr ((R * NCH <= kMaxLoads / 2 && R <= 4) || R == 1) {
      if (u8)
        launch_rows_pro<R, NCH, true, true>(grid, lds, st, a, xa);
      else
        launch_rows_pro<R, NCH, false, true>(grid, lds, st, a, xa);
      return true;
    } else if constexpr (R == 8 && NCH <= 2) {
      if (!u8) return false;
      launch_rows_pro<R, NCH, true, true>(grid, lds, st, a, xa);
      return true;
    }
  }
  return false;
}

template <int NCH>
static bool launch_rows_n(int R, bool u8, bool multi, int grid, size_t lds, hipStream_t st, const RowsArgs& a,
                          const ExclArgs* xa) {
  switch (R) {
    case 1: return launch_rows_rn<1, NCH>(u8, multi, grid, lds, st, a, xa);
    case 2: return launch_rows_rn<2, NCH>(u8, multi, grid, lds, st, a, xa);
    case 3: return launch_rows_rn<3, NCH>(u8, multi, grid, lds, st, a, xa);
    case 4: return launch_rows_rn<4, NCH>(u8, multi, grid, lds, st, a, xa);
    case 5: return launch_rows_rn<5, NCH>(u8, multi, grid, lds, st, a, xa);
    case 6: return launch_rows_rn<6, NCH>(u8, multi, grid, lds, st, a, xa);
    case 8: return launch_rows_rn<8, NCH>(u8, multi, grid, lds, st, a, xa);
    default: return false;
  }
}

static Split make_split(int total, int grid) {
  const int waves = grid * kWaves;
  return Split{total / waves, total % waves};
}

// Rows too long for a register tiling: slices of at most kSliceNch chunks per lane.
constexpr int kSliceNch = 8;
constexpr size_t kSlicedMaxLds = 144 * 1024;

// Dynamic LDS above 64 KB has to be allowed per kernel and device; frhip_init does it for the
// device it initialises, outside any stream capture.
int allow_large_lds() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&rows_sliced_kernel<kSliceNch, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSlicedMaxLds);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&rows_sliced_kernel<kSliceNch, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSlicedMaxLds);
  if (e != hipSuccess) return set_error((int)e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
  return 0;
}

// Chunks per lane and slice: the choice that wastes least, counting both the chunks of the last
// slice that lie beyond the row and the waves that get one item fewer than the others.
static size_t sliced_lds(int cs, int nslice, int rows_per_wg, bool u8) {
  const size_t padchunks = (size_t)(nslice - 1) * cs * kWave + kSliceNch * kWave;
  return padchunks * (u8 ? 64 : 16) + (size_t)rows_per_wg * nslice * sizeof(float);
}

// (among the choices whose staged vector and partial sums fit the LDS; none: *cs_out stays 0)
static void pick_slices(int total_chunks, int rows_per_wg, bool u8, int* cs_out, int* nslice_out) {
  double best = -1.0;
  *cs_out = 0;
  for (int cs = kSliceNch; cs >= 4; cs--) {
    const int nslice = (total_chunks + cs - 1) / cs;
    if (sliced_lds(cs, nslice, rows_per_wg, u8) > kSlicedMaxLds) continue;
    const long items = (long)rows_per_wg * nslice;
    const long per_wave = (items + kWaves - 1) / kWaves;
    const double eff = ((double)total_chunks / ((double)nslice * cs)) * ((double)items / (double)(per_wave * kWaves));
    if (eff > best + 1e-9) {
      best = eff;
      *cs_out = cs;
      *nslice_out = nslice;
    }
  }
}

static int launch_rows_sliced(const RowsArgs& args, bool u8, hipStream_t st, const char* what) {
  if (args.prologue != P_COPY || args.nseg != 1)
    return set_error(FRHIP_ESHAPE, "row-streaming kernel: K above 9216 (binary16) / 16384 (uint8) is supported for one matrix "
                                   "against a ready vector only");
  RowsArgs a = args;
  if (!a.res_x || !a.res_r) {
    const h1* any = reinterpret_cast<const h1*>(a.seg[0].w.data);
    if (!a.res_x && !a.res_r) a.res_n = 1;
    if (!a.res_x) a.res_x = a.res_r ? a.res_r : any;
    if (!a.res_r) a.res_r = a.res_x;
  }
  const int grid = decode_grid();
  const int N = a.seg[0].w.N;
  const int rows_per_wg = (N + grid - 1) / grid;
  SliceGeom g;
  pick_slices(chunks_per_lane(a.K, u8), rows_per_wg, u8, &g.cs, &g.nslice);
  if (g.cs == 0)
    return set_error(FRHIP_ESHAPE, "row-streaming kernel: K or N is too large for the long-row kernel's LDS (144 KB)");
  g.padchunks = (g.nslice - 1) * g.cs * kWave + kSliceNch * kWave;
  g.rows = Split{N / grid, N % grid};
  const size_t vec_bytes = (size_t)g.padchunks * (u8 ? 64 : 16);
  g.part_offset = (int)vec_bytes;
  const size_t lds = vec_bytes + (size_t)rows_per_wg * g.nslice * sizeof(float);
  if (lds > kSlicedMaxLds)
    return set_error(FRHIP_ESHAPE, "row-streaming kernel: K or N is too large for the long-row kernel's LDS (144 KB)");
  if (u8)
    hipLaunchKernelGGL((rows_sliced_kernel<kSliceNch, true>), dim3(grid), dim3(kThreads), lds, st, a, g);
  else
    hipLaunchKernelGGL((rows_sliced_kernel<kSliceNch, false>), dim3(grid), dim3(kThreads), lds, st, a, g);
  return check_launch(what);
}

static int launch_rows(const RowsArgs& args, bool u8, hipStream_t st, const char* what) {
  const int nch = round_nch(chunks_per_lane(args.K, u8));
  // the staged vector of a uint8 product takes 4 K bytes of LDS: where that and the kernel's static LDS pass 64 KB the
  // sliced kernel (which may use more) takes over
  if (nch < 0 || staged_bytes(nch, u8) + 1024 > 64 * 1024) return launch_rows_sliced(args, u8, st, what);
  static const int sliced_from = env_int("FRHIP_SLICED_FROM_K", 0);  // measurement switch: long-row kernel from this K on
  if (sliced_from > 0 && args.K >= sliced_from && args.prologue == P_COPY && args.nseg == 1)
    return launch_rows_sliced(args, u8, st, what);
  const int grid = decode_grid();
  RowsArgs a = args;
  // epilogue operands are read unconditionally: point unused ones at any readable element
  if (!a.res_x || !a.res_r) {
    const h1* any = reinterpret_cast<const h1*>(a.seg[0].w.data);
    if (!a.res_x && !a.res_r) a.res_n = 1;
    if (!a.res_x) a.res_x = a.res_r ? a.res_r : any;
    if (!a.res_r) a.res_r = a.res_x;
  }
  if (a.prologue == P_COPY && a.nseg != 1)
    return set_error(FRHIP_EINVAL, "row-streaming kernel: a staged ready vector serves one matrix");
  bool multi = false;
  const int R = pick_r(a, grid, nch, u8, &multi);
  a.bstart[0] = 0;
  for (int s = 0; s < kMaxSeg; s++)
    a.bstart[s + 1] = s < a.nseg ? a.bstart[s] + (a.seg[s].w.N + R - 1) / R : INT_MAX;
  a.split = make_split(a.bstart[a.nseg], grid);
  ExclArgs xargs;
  const ExclArgs* xa = nullptr;
  int wgs[kMaxSeg];
  if (want_exclusive(a, u8) && share_workgroups(a, R, grid, wgs)) {
    memset(&xargs, 0, sizeof(xargs));
    for (int s = 0; s < kMaxSeg; s++) {
      xargs.wg_start[s + 1] = s < a.nseg ? xargs.wg_start[s] + wgs[s] : INT_MAX;
      if (s < a.nseg) xargs.seg_split[s] = make_split(a.bstart[s + 1] - a.bstart[s], wgs[s]);
    }
    xa = &xargs;
  }
  const size_t lds = staged_bytes(nch, u8) * (u8 ? a.nseg : a.nvec);
  FR_TRY(check_lds(lds));
#ifdef FRHIP_TIMELINE
  a.tl_slot = (g_timeline_launches++) % kTlSlots;
#endif
  bool ok = false;
  switch (nch) {
    case 1: ok = launch_rows_n<1>(R, u8, multi, grid, lds, st, a, xa); break;
    case 2: ok = launch_rows_n<2>(R, u8, multi, grid, lds, st, a, xa); break;
    case 3: ok = launch_rows_n<3>(R, u8, multi, grid, lds, st, a, xa); break;
    case 4: ok = launch_rows_n<4>(R, u8, multi, grid, lds, st, a, xa); break;
    case 5: ok = launch_rows_n<5>(R, u8, multi, grid, lds, st, a, xa); break;
    case 8: ok = launch_rows_n<8>(R, u8, multi, grid, lds, st, a, xa); break;
    case 9: ok = launch_rows_n<9>(R, u8, multi, grid, lds, st, a, xa); break;
    case 16: ok = launch_rows_n<16>(R, u8, multi, grid, lds, st, a, xa); break;
    case 18: ok = launch_rows_n<18>(R, u8, multi, grid, lds, st, a, xa); break;
    default: break;
  }
  if (!ok) return set_error(FRHIP_ESHAPE, "row-streaming kernel: no compiled tiling for this shape");
  return check_launch(what);
}

static RowsArgs empty_args(int K) {
  RowsArgs a;
  memset(&a, 0, sizeof(a));
  a.K = K;
  for (int i = 0; i <= kMaxSeg; i++) a.start[i] = INT_MAX;
  return a;
}

static void add_seg(RowsArgs& a, const frhip_weight* w, int vec, int epi, void* out) {
  const int s = a.nseg;
  a.start[s] = s == 0 ? 0 : a.start[s];
  a.seg[s].w = to_wmat(w);
  a.seg[s].vec = vec;
  a.seg[s].epi = epi;
  a.seg[s].out = out;
  a.start[s + 1] = a.start[s] + w->N;
  a.nseg = s + 1;
}

static int launch_ln_mix_one(int C, const void* x, const void* sx, const void* ln_w, const void* ln_b,
                             const void* const* mix, h1* const* out, int nmix, void* xx_out, hipStream_t st) {
  LnMixOne a;
  a.C = C;
  a.nmix = nmix;
  a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  for (int i = 0; i < 4; i++) {
    a.mix[i] = i < nmix ? (const h1*)mix[i] : nullptr;
    a.out[i] = i < nmix ? out[i] : nullptr;
  }
  a.xx_out = (h1*)xx_out;
  hipLaunchKernelGGL(ln_mix_one_kernel, dim3(1), dim3(kThreads), 0, st, a);
  return check_launch("ln_mix_one");
}

// One matrix against a ready vector, with an epilogue: the building block of the operators of
// models wider than the fused kernels take.
static int product(const frhip_weight* w, const h1* vec, int epi, void* out, hipStream_t st, const char* what) {
  RowsArgs a = empty_args(w->K);
  a.prologue = P_COPY;
  a.nvec = 1;
  a.vec0 = vec;
  add_seg(a, w, 0, epi, out);
  return launch_rows(a, w->dtype == FRHIP_U8, st, what);
}

}  // namespace frhip

using namespace frhip;

extern "C" size_t frhip_decode_workspace_bytes(int C, int F) {
  // binary16 rwkv [C] | r [C] | x_mid [C] | g [C] ; fp32 k [C] | v [C] | r32 [C] ; (n_embd > 4096: four
  // mixed vectors, binary16 [C] each) ; binary16 vx [F]; each 256-byte aligned
  auto al = [](size_t n) { return (n + 255) / 256 * 256; };
  if (C <= 0 || F <= 0) return 0;
  // models wider than the fused kernels take (n_embd > 4096) also keep their four mixed vectors here
  const size_t wide = C > kFusedMaxC ? al(2 * (size_t)C) * 4 : 0;
  return al(2 * (size_t)C) * 4 + al(2 * (size_t)F) + al(4 * (size_t)C) * 3 + wide;
}

namespace {
struct Workspace {
  h1 *rwkv, *r, *vx, *xmid, *g;
  float *k32, *v32, *r32;
  h1* mixed[4];  // n_embd > 4096 only
};
Workspace carve(void* ws, int C) {
  auto al = [](size_t n) { return (n + 255) / 256 * 256; };
  unsigned char* p = static_cast<unsigned char*>(ws);
  Workspace w;
  w.rwkv = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.r = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.xmid = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.g = reinterpret_cast<h1*>(p);
  p += al(2 * (size_t)C);
  w.k32 = reinterpret_cast<float*>(p);
  p += al(4 * (size_t)C);
  w.v32 = reinterpret_cast<float*>(p);
  p += al(4 * (size_t)C);
  w.r32 = reinterpret_cast<float*>(p);
  p += al(4 * (size_t)C);
  for (int i = 0; i < 4; i++) {
    w.mixed[i] = reinterpret_cast<h1*>(p);
    if (C > kFusedMaxC) p += al(2 * (size_t)C);
  }
  w.vx = reinterpret_cast<h1*>(p);  // [F], the only part whose size the attention operators do not know: last
  return w;
}
}  // namespace

// ---------------------------------------------------------------------------
// Scratch for frhip_ffn_one_static: the workspace of frhip_ffn_one for the largest shape
// that entry point accepts, as a file-scope device array.  Every GPU the library runs on holds
// its own copy (112 KB) until the process ends.  Host code never uses the array's name as an
// address: the device address is looked up once per device with hipGetSymbolAddress and kept.
// ---------------------------------------------------------------------------
namespace frhip {
constexpr int kStaticMaxC = 4096;
constexpr int kStaticMaxF = 16384;
// frhip_decode_workspace_bytes(kStaticMaxC, kStaticMaxF): 4 x 8 KB + 32 KB + 3 x 16 KB
constexpr size_t kStaticScratchBytes = 4 * 8192 + 32768 + 3 * 16384;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, once looked up
static std::mutex g_scratch_mu;

// Looks up the current device's copy of `scratch` (once per device) and returns it in *ptr.
int static_scratch(void** ptr) {
  int dev = -1;
  FR_TRY(hip_result(hipGetDevice(&dev), "hipGetDevice"));
  if (dev < 0 || dev >= kMaxDevices) return set_error(FRHIP_EINVAL, "device index beyond the static scratch table");
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    FR_TRY(hip_result(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"));
    if (!p || reinterpret_cast<uintptr_t>(p) % 256 != 0) return set_error(FRHIP_ESTATE, "static scratch has no usable device address");
    g_scratch_ptr[dev] = p;
  }
  if (ptr) *ptr = g_scratch_ptr[dev];
  return 0;
}
}  // namespace frhip

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
  Workspace w = carve(workspace, C);
  const int grid = decode_grid();

  if (C > kFusedMaxC) {
    const void* mixes[3] = {k_mix, v_mix, r_mix};
    FR_TRY(launch_ln_mix_one(C, x, sx, ln_w, ln_b, mixes, w.mixed, 3, xx_out, st));
    FR_TRY(product(kw, w.mixed[0], E_STORE_F32, w.k32, st, "att_k"));
    FR_TRY(product(vw, w.mixed[1], E_STORE_F32, w.v32, st, "att_v"));
    FR_TRY(product(rw, w.mixed[2], E_SIGMOID, w.r, st, "att_r"));
    Wkv4One q;
    q.C = C;
    q.k = w.k32; q.v = w.v32; q.aa = aa; q.bb = bb; q.pp = pp; q.td = t_decay; q.tf = t_first;
    q.r = w.r; q.rwkv_out = w.rwkv;
    q.aa_out = aa_out; q.bb_out = bb_out; q.pp_out = pp_out;
    hipLaunchKernelGGL(wkv4_one_kernel, dim3((C + 255) / 256), dim3(256), 0, st, q);
    FR_TRY(check_launch("wkv4_one"));
    RowsArgs b = empty_args(C);
    b.prologue = P_COPY;
    b.nvec = 1;
    b.vec0 = w.rwkv;
    b.res_x = (const h1*)x;
    b.res_n = C;
    add_seg(b, ow, 0, E_RESIDUAL, x_out);
    return launch_rows(b, ow->dtype == FRHIP_U8, st, "att_out");
  }

  AttFrontV4 a;
  a.C = C;
  a.split = make_split(C, grid);
  a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  a.mk = (const h1*)k_mix; a.mv = (const h1*)v_mix; a.mr = (const h1*)r_mix;
  a.aa = aa; a.bb = bb; a.pp = pp; a.td = t_decay; a.tf = t_first;
  a.kw = to_wmat(kw); a.vw = to_wmat(vw); a.rw = to_wmat(rw);
  a.xx_out = (h1*)xx_out; a.rwkv_out = w.rwkv;
  a.aa_out = aa_out; a.bb_out = bb_out; a.pp_out = pp_out;
  const bool u8 = kw->dtype == FRHIP_U8;
  const int nch = chunks_per_lane(C, u8);  // C <= 4096: at most 8 (fp16) or 4 (uint8)
  const int nch_t = nch <= 1 ? 1 : nch == 2 ? 2 : nch <= 4 ? 4 : nch == 5 ? 5 : 8;  // compiled tilings
  const size_t lds = staged_bytes(nch_t, u8) * 3;
  FR_TRY(check_lds(lds));
  // uint8 weights, more channels than one workgroup per CU has waves (n_embd 2560 ... 4096): one channel
  // per wave over up to two workgroups per CU instead of a loop over two channels in some waves.  The loop's
  // second set of uint8 rows does not fit the registers beside the first, so its loads wait for the first
  // channel's products (decode of the 3B / 7B widths: 2452 -> 2714, 1704 -> 1906 tok/s over 8 layers; the
  // binary16 loop, which requests ahead, is as fast or faster than two workgroups: 2696 vs 2625 tok/s).
  static const bool two_wgs = env_int("FRHIP_ATT_TWO_WGS", 1) == 1;
  int grid_a = grid;
  if (two_wgs && u8 && C > grid * kWaves && C <= 2 * grid * kWaves) grid_a = (C + kWaves - 1) / kWaves;
  const bool single = C <= grid_a * kWaves;
  a.split = make_split(C, grid_a);
#define FR_ATT_FRONT(N)                                                                                     \
  do {                                                                                                      \
    if (u8 && single)                                                                                       \
      hipLaunchKernelGGL((att_front_v4_kernel<N, true, true>), dim3(grid_a), dim3(kThreads), lds, st, a);   \
    else if (u8)                                                                                            \
      hipLaunchKernelGGL((att_front_v4_kernel<N, true, false>), dim3(grid_a), dim3(kThreads), lds, st, a);  \
    else if (single)                                                                                        \
      hipLaunchKernelGGL((att_front_v4_kernel<N, false, true>), dim3(grid_a), dim3(kThreads), lds, st, a);  \
    else                                                                                                    \
      hipLaunchKernelGGL((att_front_v4_kernel<N, false, false>), dim3(grid_a), dim3(kThreads), lds, st, a); \
  } while (0)
  if (nch <= 1) FR_ATT_FRONT(1);
  else if (nch == 2) FR_ATT_FRONT(2);
  else if (nch <= 4) FR_ATT_FRONT(4);
  else if (nch == 5) FR_ATT_FRONT(5);
  else FR_ATT_FRONT(8);
#undef FR_ATT_FRONT
  FR_TRY(check_launch("att_front_v4"));

  RowsArgs b = empty_args(C);
  b.prologue = P_COPY;
  b.nvec = 1;
  b.vec0 = w.rwkv;
  b.res_x = (const h1*)x;
  b.res_n = C;
  add_seg(b, ow, 0, E_RESIDUAL, x_out);
  return launch_rows(b, ow->dtype == FRHIP_U8, st, "att_out");
}

// Shared by RWKV-5.0 (no gate: g_mix and gw null, u and w per head) and RWKV-5.1/5.2.
static int att_one_v5_impl(bool v50, int C, int H, const void* x, const void* sx, const float* s, const void* ln_w,
                                  const void* ln_b, const float* lx_w, const float* lx_b, const void* k_mix,
                                  const void* v_mix, const void* r_mix, const void* g_mix, const float* t_decay,
                                  const float* t_first, const frhip_weight* kw, const frhip_weight* vw,
                                  const frhip_weight* rw, const frhip_weight* gw, const frhip_weight* ow,
                                  void* x_out, void* xx_out, float* s_out, void* workspace, frhip_stream s_) {
  FR_TRY(check_embd(C));
  if (H <= 0 || C % H != 0 || C / H != 64) return set_error(FRHIP_ESHAPE, "att_one_v5: head size must be 64");
  FR_TRY(check_vec(x, "x is null or misaligned"));
  FR_TRY(check_vec(sx, "sx is null or misaligned"));
  FR_TRY(check_vec(ln_w, "ln_w is null or misaligned"));
  FR_TRY(check_vec(ln_b, "ln_b is null or misaligned"));
  FR_TRY(check_vec(k_mix, "k_mix is null or misaligned"));
  FR_TRY(check_vec(v_mix, "v_mix is null or misaligned"));
  FR_TRY(check_vec(r_mix, "r_mix is null or misaligned"));
  if (!v50) FR_TRY(check_vec(g_mix, "g_mix is null or misaligned"));
  FR_TRY(check_vec(x_out, "x_out is null or misaligned"));
  FR_TRY(check_vec(xx_out, "xx_out is null or misaligned"));
  FR_TRY(check_vec(workspace, "workspace is null or misaligned"));
  if (!s || !s_out || !lx_w || !lx_b || !t_decay || !t_first) return set_error(FRHIP_EINVAL, "att_one_v5: null state or parameter");
  if (xx_out == sx) return set_error(FRHIP_EINVAL, "att_one_v5: xx_out must not alias sx");
  FR_TRY(check_weight(kw, C, C));
  FR_TRY(check_weight(vw, C, C));
  FR_TRY(check_weight(rw, C, C));
  if (!v50) FR_TRY(check_weight(gw, C, C));
  FR_TRY(check_weight(ow, C, C));
  if (kw->dtype != vw->dtype || kw->dtype != rw->dtype || (!v50 && kw->dtype != gw->dtype))
    return set_error(FRHIP_EINVAL, "att_one_v5: key/value/receptance/gate dtypes differ");
  hipStream_t st = static_cast<hipStream_t>(s_);
  Workspace w = carve(workspace, C);

  // LN -> 4 mixes -> k, v, r (fp32) and g = silu(.) (half)      att.cu:276-290
  if (C > kFusedMaxC) {
    const void* mixes[4] = {k_mix, v_mix, r_mix, g_mix};
    FR_TRY(launch_ln_mix_one(C, x, sx, ln_w, ln_b, mixes, w.mixed, v50 ? 3 : 4, xx_out, st));
    FR_TRY(product(kw, w.mixed[0], E_STORE_F32, w.k32, st, "att_v5_k"));
    FR_TRY(product(vw, w.mixed[1], E_STORE_F32, w.v32, st, "att_v5_v"));
    FR_TRY(product(rw, w.mixed[2], E_STORE_F32, w.r32, st, "att_v5_r"));
    if (!v50) FR_TRY(product(gw, w.mixed[3], E_SILU, w.g, st, "att_v5_g"));
  } else {
    RowsArgs a = empty_args(C);
    a.prologue = P_LN_MIX;
    a.nvec = v50 ? 3 : 4;
    a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
    a.mix[0] = (const h1*)k_mix; a.mix[1] = (const h1*)v_mix; a.mix[2] = (const h1*)r_mix; a.mix[3] = (const h1*)g_mix;
    a.xx_out = (h1*)xx_out;
    add_seg(a, kw, 0, E_STORE_F32, w.k32);
    add_seg(a, vw, 1, E_STORE_F32, w.v32);
    add_seg(a, rw, 2, E_STORE_F32, w.r32);
    if (!v50) add_seg(a, gw, 3, E_SILU, w.g);
    FR_TRY(launch_rows(a, kw->dtype == FRHIP_U8, st, "att_v5_front"));
  }

  Wkv5One k;
  k.H = H;
  k.uw_head = v50 ? 1 : 0;
  k.s = s; k.r = w.r32; k.k = w.k32; k.v = w.v32; k.w = t_decay; k.u = t_first; k.lx_w = lx_w; k.lx_b = lx_b;
  k.g = v50 ? nullptr : w.g; k.s_out = s_out; k.gated_out = w.rwkv;
  hipLaunchKernelGGL(wkv5_one_kernel, dim3(H), dim3(256), 0, st, k);
  FR_TRY(check_launch("wkv5_one"));

  RowsArgs b = empty_args(C);
  b.prologue = P_COPY;
  b.nvec = 1;
  b.vec0 = w.rwkv;
  b.res_x = (const h1*)x;
  b.res_n = C;
  add_seg(b, ow, 0, E_RESIDUAL, x_out);
  return launch_rows(b, ow->dtype == FRHIP_U8, st, "att_v5_out");
}

extern "C" int frhip_att_one_v5_1(int C, int H, const void* x, const void* sx, const float* s, const void* ln_w,
                                  const void* ln_b, const float* lx_w, const float* lx_b, const void* k_mix,
                                  const void* v_mix, const void* r_mix, const void* g_mix, const float* t_decay,
                                  const float* t_first, const frhip_weight* kw, const frhip_weight* vw,
                                  const frhip_weight* rw, const frhip_weight* gw, const frhip_weight* ow,
                                  void* x_out, void* xx_out, float* s_out, void* workspace, frhip_stream s_) {
  return att_one_v5_impl(false, C, H, x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay, t_first,
                         kw, vw, rw, gw, ow, x_out, xx_out, s_out, workspace, s_);
}

// att_one_v5 (RWKV-5.0): kernels/cuda/att.cu:219-265,362-391.
extern "C" int frhip_att_one_v5(int C, int H, const void* x, const void* sx, const float* s, const void* ln_w,
                                const void* ln_b, const float* lx_w, const float* lx_b, const void* k_mix,
                                const void* v_mix, const void* r_mix, const float* t_decay, const float* t_first,
                                const frhip_weight* kw, const frhip_weight* vw, const frhip_weight* rw,
                                const frhip_weight* ow, void* x_out, void* xx_out, float* s_out, void* workspace,
                                frhip_stream s_) {
  return att_one_v5_impl(true, C, H, x, sx, s, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, nullptr, t_decay, t_first,
                         kw, vw, rw, nullptr, ow, x_out, xx_out, s_out, workspace, s_);
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
  Workspace w = carve(workspace, C);

  if (C > kFusedMaxC) {
    const void* mixes[2] = {r_mix, k_mix};
    FR_TRY(launch_ln_mix_one(C, x, sx, ln_w, ln_b, mixes, w.mixed, 2, xx_out, st));
    FR_TRY(product(rw, w.mixed[0], E_SIGMOID, w.r, st, "ffn_r"));
    FR_TRY(product(kw, w.mixed[1], E_RELU2, w.vx, st, "ffn_k"));
  } else {
    RowsArgs a = empty_args(C);
    a.prologue = P_LN_MIX;
    a.nvec = 2;
    a.x = (const h1*)x; a.sx = (const h1*)sx; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
    a.mix[0] = (const h1*)r_mix;
    a.mix[1] = (const h1*)k_mix;
    a.xx_out = (h1*)xx_out;
    add_seg(a, rw, 0, E_SIGMOID, w.r);
    add_seg(a, kw, 1, E_RELU2, w.vx);
    FR_TRY(launch_rows(a, kw->dtype == FRHIP_U8, st, "ffn_front"));
  }

  RowsArgs b = empty_args(F);
  b.prologue = P_COPY;
  b.nvec = 1;
  b.vec0 = w.vx;
  b.res_x = (const h1*)x;
  b.res_n = C;
  b.res_r = w.r;
  b.div2 = post_div2 ? 1 : 0;
  add_seg(b, vw, 0, E_FFN_OUT, x_out);
  return launch_rows(b, vw->dtype == FRHIP_U8, st, "ffn_out");
}

extern "C" int frhip_ffn_one_static(int C, int F, const void* x, const void* sx, const void* ln_w, const void* ln_b,
                                    const void* k_mix, const void* r_mix, const frhip_weight* kw,
                                    const frhip_weight* vw, const frhip_weight* rw, void* x_out, void* xx_out,
                                    int post_div2, frhip_stream s) {
  if (C > kStaticMaxC || F > kStaticMaxF)
    return set_error(FRHIP_ESHAPE, "ffn_one_static: n_embd above 4096 or n_ffn above 16384 exceeds the built-in scratch; "
                                   "use frhip_ffn_one with a workspace");
  void* ws = nullptr;
  FR_TRY(static_scratch(&ws));
  // r [C] and relu(k)^2 [F] are written in full by the first launch before the second reads them:
  // nothing in the scratch has to start at zero, whatever an earlier (larger) call left there.
  return frhip_ffn_one(C, F, x, sx, ln_w, ln_b, k_mix, r_mix, kw, vw, rw, x_out, xx_out, post_div2, ws, s);
}

extern "C" int frhip_head(int C, const void* x, const void* ln_w, const void* ln_b, const frhip_weight* head,
                          float* logits, frhip_stream s) {
  return frhip_head_mirror(C, x, ln_w, ln_b, head, logits, nullptr, s);
}

extern "C" int frhip_head_mirror(int C, const void* x, const void* ln_w, const void* ln_b, const frhip_weight* head,
                                 float* logits, float* mirror, frhip_stream s) {
  FR_TRY(check_embd(C));
  FR_TRY(check_vec(x, "x is null or misaligned"));
  FR_TRY(check_vec(ln_w, "ln_w is null or misaligned"));
  FR_TRY(check_vec(ln_b, "ln_b is null or misaligned"));
  if (!logits) return set_error(FRHIP_EINVAL, "logits is null");
  FR_TRY(check_weight(head, C, 0));
  RowsArgs a = empty_args(C);
  a.prologue = P_LN;
  a.nvec = 1;
  a.x = (const h1*)x; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  a.mirror = mirror;
  add_seg(a, head, 0, E_LOGITS, logits);
  return launch_rows(a, head->dtype == FRHIP_U8, static_cast<hipStream_t>(s), "head");
}

extern "C" int frhip_gemv(const void* x, const frhip_weight* w, void* y, int out_dtype, frhip_stream s) {
  FR_TRY(check_vec(x, "x is null or misaligned"));
  if (!y) return set_error(FRHIP_EINVAL, "y is null");
  if (out_dtype != FRHIP_F16 && out_dtype != FRHIP_F32) return set_error(FRHIP_EINVAL, "gemv: out_dtype must be F16 or F32");
  FR_TRY(check_weight(w, 0, 0));
  RowsArgs a = empty_args(w->K);
  a.prologue = P_COPY;
  a.nvec = 1;
  a.vec0 = (const h1*)x;
  add_seg(a, w, 0, out_dtype == FRHIP_F32 ? E_STORE_F32 : E_STORE_F16, y);
  return launch_rows(a, w->dtype == FRHIP_U8, static_cast<hipStream_t>(s), "gemv");
}

#ifdef FRHIP_TIMELINE
// Measurement build only: copies the timestamps of the last 8 row-kernel launches to `dst`
// ([8 slots][4096 waves][16] uint64, 100 MHz ticks; launch number n took slot n % 8) and reports how many
// launches have taken a slot so far.
extern "C" int frhip_timeline_read(void* dst, int* launches) {
  *launches = frhip::g_timeline_launches;
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(frhip::g_timeline), sizeof(frhip::g_timeline));
}
#endif
