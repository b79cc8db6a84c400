// Seq-mode (prompt) operators: layernorm + token shift + mix over T rows, the WKV scans of
// RWKV-4 and RWKV-5.2, and the att_seq / ffn_seq compositions around the MFMA GEMM.
//
// Both recurrences are linear in their state, so the scans run CHUNKED over time instead of
// as one serial loop of T steps on a handful of wavefronts (kernels/cuda/att_seq.cu:258-322
// runs 64 threads per head for T steps):
//   1. every chunk is scanned from an EMPTY state, all chunks in parallel -> local end states;
//   2. a short serial pass over the chunks turns local end states into the true state at the
//      start of every chunk (state_in[c+1] = decay^len(state_in[c]) + local[c]);
//   3. every chunk is scanned again from its true start state, all chunks in parallel,
//      producing the outputs; the last chunk leaves the final state.
// The arithmetic of pass 3 is the one-token recurrence (kernels/cuda/att.cu:30-62, :64-81);
// only the representation of the carried state differs from a serial scan, at fp32 rounding level.
#include <climits>
#include <cstring>

#include "gemm.h"

#pragma clang fp contract(off)

namespace frhip {

// ---------------------------------------------------------------------------
// layernorm + token shift + mix for T rows: one workgroup (256 threads) per row.
//   xx_t = LN(x_t) ; sx_t = (t == 0) ? state : xx_{t-1} ; out_i[t] = mix(xx_t, sx_t, mix_i)
// (kernels/cuda/ffn_seq.cu:70-77, att_seq.cu:379-389).  LN(x_{t-1}) is recomputed by the
// workgroup of row t, which saves a [T, C] round trip.  Row T-1 also writes xx_{T-1}, the
// new shift state.
// ---------------------------------------------------------------------------
struct LnMixSeq {
  int T, C, nmix;
  const h1 *x, *state, *ln_w, *ln_b;
  const h1* mix[4];
  h1* out[4];
  h1* xx_last;
};

__device__ __forceinline__ void ln_row_to_lds(const h1* xr, const h1* g, const h1* b, int C, h1* dst, float* red) {
  float s = 0.f;
  for (int i = threadIdx.x; i < C; i += 256) s += (float)xr[i];
  const float mean = block_sum<4>(s, red) / (float)C;
  float q = 0.f;
  for (int i = threadIdx.x; i < C; i += 256) {
    float d = (float)xr[i] - mean;
    q += d * d;
  }
  float var = block_sum<4>(q, red) / (float)C;
  var = var > 0.f ? var : 0.f;
  const float inv = 1.0f / sqrtf(var + 1e-5f);
  for (int i = threadIdx.x; i < C; i += 256) {
    h1 n = (h1)(((float)xr[i] - mean) * inv);
    dst[i] = (n * g[i]) + b[i];
  }
}

__global__ __launch_bounds__(256) void ln_mix_seq_kernel(LnMixSeq a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  __shared__ float red[4];
  h1* cur = reinterpret_cast<h1*>(smem);
  h1* prev = cur + a.C;
  const int t = blockIdx.x, C = a.C;
  ln_row_to_lds(a.x + (size_t)t * C, a.ln_w, a.ln_b, C, cur, red);
  if (t == 0) {
    for (int i = threadIdx.x; i < C; i += 256) prev[i] = a.state[i];
  } else {
    ln_row_to_lds(a.x + (size_t)(t - 1) * C, a.ln_w, a.ln_b, C, prev, red);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < C; i += 256) {
    const h1 xx = cur[i], sx = prev[i];
    for (int m = 0; m < a.nmix; m++) a.out[m][(size_t)t * C + i] = mix1(xx, sx, a.mix[m][i]);
    if (t == a.T - 1) a.xx_last[i] = xx;
  }
}

// The same for C % 8 == 0, C <= 8 * 256 * NG: a workgroup takes kLnRows consecutive rows plus the
// row before them (the token shift of its first row), every thread owns NG groups of 8 elements
// of every row in registers, all rows are loaded up front and their statistics reduced together
// (two barriers per workgroup), and the mixed rows leave as 16-byte stores.  The launch is a chain
// of one load, two reductions and one store per workgroup, so what counts is how many workgroups
// a compute unit has to overlap: at T = 1024, C = 2048 four rows per workgroup (one workgroup per
// CU, every row read 1.25 times) take 8.7 us, two 7.4 us, one (every row read twice) 7.0 us.
constexpr int kLnRows = 1;

template <int NG>
__global__ __launch_bounds__(256) void ln_mix_rows_kernel(LnMixSeq a) {
  constexpr int NR = kLnRows + 1;  // row 0 is the row before the workgroup's first
  __shared__ float red[2][4][NR];
  const int C = a.C, ngrp = C >> 3;
  const int t0 = blockIdx.x * kLnRows;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  h8 xr[NR][NG], gam[NG], bet[NG];
  bool own[NG];
#pragma unroll
  for (int n = 0; n < NG; n++) {
    const int g = threadIdx.x + n * 256;
    own[n] = g < ngrp;
    const int gc = own[n] ? g : 0;
#pragma unroll
    for (int r = 0; r < NR; r++) {
      int t = t0 - 1 + r;
      t = t < 0 ? 0 : (t < a.T ? t : a.T - 1);
      xr[r][n] = reinterpret_cast<const h8*>(a.x + (size_t)t * C)[gc];
    }
    gam[n] = reinterpret_cast<const h8*>(a.ln_w)[gc];
    bet[n] = reinterpret_cast<const h8*>(a.ln_b)[gc];
  }
  h8 shift0[NG];  // the shift state, used instead of LN(row -1) by the first workgroup
  if (t0 == 0) {
#pragma unroll
    for (int n = 0; n < NG; n++) shift0[n] = reinterpret_cast<const h8*>(a.state)[own[n] ? threadIdx.x + n * 256 : 0];
  }
  float mean[NR], inv[NR];
  {
    float s[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
      s[r] = 0.f;
#pragma unroll
      for (int n = 0; n < NG; n++)
        if (own[n])
#pragma unroll
          for (int i = 0; i < 8; i++) s[r] += (float)xr[r][n][i];
      s[r] = wave_sum(s[r]);
      if (lane == 0) red[0][wv][r] = s[r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; r++) mean[r] = (((red[0][0][r] + red[0][1][r]) + red[0][2][r]) + red[0][3][r]) / (float)C;
    float q[NR];
#pragma unroll
    for (int r = 0; r < NR; r++) {
      q[r] = 0.f;
#pragma unroll
      for (int n = 0; n < NG; n++)
        if (own[n])
#pragma unroll
          for (int i = 0; i < 8; i++) {
            const float d = (float)xr[r][n][i] - mean[r];
            q[r] += d * d;
          }
      q[r] = wave_sum(q[r]);
      if (lane == 0) red[1][wv][r] = q[r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; r++) {
      float var = (((red[1][0][r] + red[1][1][r]) + red[1][2][r]) + red[1][3][r]) / (float)C;
      var = var > 0.f ? var : 0.f;
      inv[r] = 1.0f / sqrtf(var + 1e-5f);
    }
  }
#pragma unroll
  for (int n = 0; n < NG; n++) {
    if (!own[n]) continue;
    const int g = threadIdx.x + n * 256;
    h8 prev;
#pragma unroll
    for (int r = 0; r < NR; r++) {
      h8 xx;
#pragma unroll
      for (int i = 0; i < 8; i++) {  // kernels/cuda/layer_norm.cu:60-69: half, * gamma in half, + beta in half
        const h1 nrm = (h1)(((float)xr[r][n][i] - mean[r]) * inv[r]);
        xx[i] = (nrm * gam[n][i]) + bet[n][i];
      }
      if (r == 0) {
        prev = t0 == 0 ? shift0[n] : xx;
        continue;
      }
      const int t = t0 + r - 1;
      if (t < a.T) {
        for (int m = 0; m < a.nmix; m++) {
          const h8 mx = reinterpret_cast<const h8*>(a.mix[m])[g];
          h8 o;
#pragma unroll
          for (int i = 0; i < 8; i++) o[i] = mix1(xx[i], prev[i], mx[i]);
          reinterpret_cast<h8*>(a.out[m] + (size_t)t * C)[g] = o;
        }
        if (t == a.T - 1) reinterpret_cast<h8*>(a.xx_last)[g] = xx;
      }
      prev = xx;
    }
  }
}

// ---------------------------------------------------------------------------
// RWKV-4 WKV scan.  k, v [T][C] fp32; r [T][C] half (already through the sigmoid),
// overwritten with r * half(wkv).
// ---------------------------------------------------------------------------
struct Wkv4Seq {
  int T, C, Lc, nchunk;
  const float *k, *v, *u, *w;
  h1* r;
  const float *aa, *bb, *pp;  // state before the sequence (read by pass 1 only; may alias aa_out / bb_out / pp_out)
  float *la, *lb, *lp;        // [nchunk][C] local end states (pass 1)
  float *sa, *sb, *sp;        // [nchunk][C] state at the start of each chunk (row 0: pass 1; the rest: the serial pass)
  float *aa_out, *bb_out, *pp_out;
};

// Steps per batch of loads in the chunk passes: a thread requests the k, v (and r) of kScanB steps
// before the recurrence touches the first, so a chunk of 16 steps costs one memory round trip
// instead of 16 (with two waves per SIMD little else hides them: 8.3 -> 6.9 us and 10.7 -> 9.0 us
// per launch at T = 1024).  What remains is launch, one round trip and the library expf (~28 VALU
// instructions; three per token and channel over the passes, one per pair: exp_pair below); a
// six-instruction exp2-based exponential within 2 ulp was measured when the passes still took six
// (28.4 -> 25.2 us) and was not kept: the passes then no longer compute exactly what the one-token
// kernel does.
constexpr int kScanB = 16;

// p = max(a, b) (b on ties), ea = exp(a - p), eb = exp(b - p) with one exponential instead of two: the
// argument of the other one is +0 and expf(+0) is exactly 1, so for finite a and b these are the bits
// of the two calls.
__device__ __forceinline__ void exp_pair(float a, float b, float& p, float& ea, float& eb) {
  const bool first = a > b;
  p = first ? a : b;
  const float e = expf(first ? b - a : a - b);
  ea = first ? 1.0f : e;
  eb = first ? e : 1.0f;
}

__global__ __launch_bounds__(256) void wkv4_local_kernel(Wkv4Seq a) {
  const int c = blockIdx.x * 256 + threadIdx.x, ch = blockIdx.y;
  if (c >= a.C) return;
  const int t0 = ch * a.Lc, t1 = min(t0 + a.Lc, a.T);
  const float w = a.w[c];
  float aa = 0.f, bb = 0.f, pp = -1e30f;
  for (int tb = t0; tb < t1; tb += kScanB) {
    float kk[kScanB], vv[kScanB];
#pragma unroll
    for (int i = 0; i < kScanB; i++) {
      const int t = tb + i < t1 ? tb + i : t1 - 1;
      kk[i] = a.k[(size_t)t * a.C + c];
      vv[i] = a.v[(size_t)t * a.C + c];
    }
#pragma unroll
    for (int i = 0; i < kScanB; i++) {
      if (tb + i < t1) {
        const float k = kk[i], v = vv[i];
        float p, e1, e2;
        exp_pair(w + pp, k, p, e1, e2);
        aa = e1 * aa + e2 * v;
        bb = e1 * bb + e2;
        pp = p;
      }
    }
  }
  const size_t o = (size_t)ch * a.C + c;
  a.la[o] = aa;
  a.lb[o] = bb;
  a.lp[o] = pp;
  // The state before the sequence is copied into chunk 0's start-state slot.  The later passes read it
  // from there, never from aa / bb / pp: the last chunk of the apply pass writes aa_out / bb_out / pp_out,
  // which may be the same buffers, while chunks that were scheduled later have not started yet.
  if (ch == 0) {
    a.sa[c] = a.aa[c];
    a.sb[c] = a.bb[c];
    a.sp[c] = a.pp[c];
  }
}

// The serial pass over the chunks.  A channel's step needs three values per chunk; they are read
// eight chunks at a time ahead of the recurrence, so the pass costs one memory round trip per
// eight chunks instead of one per chunk.
__global__ __launch_bounds__(64) void wkv4_carry_kernel(Wkv4Seq a) {
  const int c = blockIdx.x * 64 + threadIdx.x;
  if (c >= a.C) return;
  constexpr int PF = 8;
  const float w = a.w[c];
  float aa = a.sa[c], bb = a.sb[c], pp = a.sp[c];  // the incoming state, left there by wkv4_local_kernel
  for (int ch0 = 0; ch0 < a.nchunk; ch0 += PF) {
    float lp[PF], la[PF], lb[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int ch = ch0 + i < a.nchunk ? ch0 + i : a.nchunk - 1;
      const size_t o = (size_t)ch * a.C + c;
      lp[i] = a.lp[o];
      la[i] = a.la[o];
      lb[i] = a.lb[o];
    }
#pragma unroll
    for (int i = 0; i < PF; i++) {
      const int ch = ch0 + i;
      if (ch < a.nchunk) {
        const size_t o = (size_t)ch * a.C + c;
        a.sa[o] = aa;
        a.sb[o] = bb;
        a.sp[o] = pp;
        const int len = min(a.Lc, a.T - ch * a.Lc);
        // the incoming state decays by len steps; the chunk's own tokens contribute its local state
        float p, e1, e2;
        exp_pair(pp + (float)len * w, lp[i], p, e1, e2);
        aa = e1 * aa + e2 * la[i];
        bb = e1 * bb + e2 * lb[i];
        pp = p;
      }
    }
  }
}

// CARRY: the chunk forms its own start state by composing, in order, the incoming state with the
// local end states of the chunks before it -- the serial pass's arithmetic, step for step, so the
// results are the serial pass's bit for bit -- instead of reading what wkv4_carry_kernel left.  Chunk j
// spends j compositions (two exponentials each) where the serial pass spends one launch and nchunk
// dependent steps per channel; the local states are requested eight chunks at a time.
template <bool CARRY>
__global__ __launch_bounds__(256) void wkv4_apply_kernel(Wkv4Seq a) {
  // the chunks with the longest prefix first: they decide when the launch ends
  const int c = blockIdx.x * 256 + threadIdx.x, ch = CARRY ? (int)(gridDim.y - 1 - blockIdx.y) : (int)blockIdx.y;
  if (c >= a.C) return;
  const int t0 = ch * a.Lc, t1 = min(t0 + a.Lc, a.T);
  const float w = a.w[c], u = a.u[c];
  const size_t o = (size_t)ch * a.C + c;
  float aa, bb, pp;
  if constexpr (CARRY) {
    constexpr int PF = 8;
    aa = a.sa[c], bb = a.sb[c], pp = a.sp[c];  // the incoming state, left there by wkv4_local_kernel
    const float pdw = (float)a.Lc * w;  // every chunk before this one is a full chunk
    for (int j0 = 0; j0 < ch; j0 += PF) {
      float lp[PF], la[PF], lb[PF];
#pragma unroll
      for (int i = 0; i < PF; i++) {
        const int j = j0 + i < ch ? j0 + i : ch - 1;
        const size_t q = (size_t)j * a.C + c;
        lp[i] = a.lp[q];
        la[i] = a.la[q];
        lb[i] = a.lb[q];
      }
#pragma unroll
      for (int i = 0; i < PF; i++) {
        if (j0 + i < ch) {
          float p, e1, e2;
          exp_pair(pp + pdw, lp[i], p, e1, e2);
          aa = e1 * aa + e2 * la[i];
          bb = e1 * bb + e2 * lb[i];
          pp = p;
        }
      }
    }
  } else {
    aa = a.sa[o], bb = a.sb[o], pp = a.sp[o];
  }
  for (int tb = t0; tb < t1; tb += kScanB) {
    float kk[kScanB], vv[kScanB];
    h1 rr[kScanB];
#pragma unroll
    for (int i = 0; i < kScanB; i++) {
      const int t = tb + i < t1 ? tb + i : t1 - 1;
      const size_t j = (size_t)t * a.C + c;
      kk[i] = a.k[j];
      vv[i] = a.v[j];
      rr[i] = a.r[j];
    }
#pragma unroll
    for (int i = 0; i < kScanB; i++) {
      if (tb + i < t1) {
        const float k = kk[i], v = vv[i];
        // kernels/cuda/att.cu:43-60
        float p, e1, e2;
        exp_pair(pp, u + k, p, e1, e2);
        const float wkv = (e1 * aa + e2 * v) / (e1 * bb + e2);
        a.r[(size_t)(tb + i) * a.C + c] = rr[i] * (h1)wkv;
        exp_pair(w + pp, k, p, e1, e2);
        aa = e1 * aa + e2 * v;
        bb = e1 * bb + e2;
        pp = p;
      }
    }
  }
  if (ch == a.nchunk - 1) {
    a.aa_out[c] = aa;
    a.bb_out[c] = bb;
    a.pp_out[c] = pp;
  }
}

// ---------------------------------------------------------------------------
// RWKV-5.2 scan, head size 64.  r, k, v [T][C] fp32; state [H][64 key][64 value] fp32.
// A workgroup of 256 threads serves one (head, chunk): thread t owns value index
// j = t % 64 and key rows i = (t / 64) * 16 .. +15 of the state (16 registers).
// Output row t: y_j = sum_i r_i (u_i k_i v_j + s_ij), then groupnorm over the head's 64
// values, rounding to half and the gate multiply (att_seq.cu:294-316, :406-411).
// The scan over a prompt regroups the sums by chunk anyway, so its multiply-adds are fused (four
// instructions per state element and step instead of seven); the one-token operator keeps the
// separately rounded products and sums.  The partial sums of 16 steps wait in LDS for one round
// of group norms shared by the four waves, instead of a barrier and one wave's group norm per step.
// ---------------------------------------------------------------------------
struct Wkv5Seq {
  int T, C, H, Lc, nchunk;
  int uw_head;       // 0: u, w are [H][64] (RWKV-5.2); 1: one value per head (RWKV-5.0)
  const float *r, *k, *v, *w, *u, *lx_w, *lx_b;
  const h1* g;       // [T][C] gate, already through silu; null for RWKV-5.0
  const float* s;    // state before the sequence
  float* loc;        // [nchunk][H][64][64] local end states
  float* sin;        // [nchunk][H][64][64] state at the start of each chunk
  float* s_out;
  h1* gated;         // [T][C]
};

constexpr int S5 = 64;

__global__ __launch_bounds__(256) void wkv5_local_kernel(Wkv5Seq a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* kk = reinterpret_cast<float*>(smem);  // [Lc][64]
  float* vv = kk + a.Lc * S5;
  __shared__ float wsh[S5];
  const int h = blockIdx.x, ch = blockIdx.y, t = threadIdx.x, j = t & 63, ig = t >> 6;
  const int t0 = ch * a.Lc, len = min(a.Lc, a.T - t0);
  for (int e = t; e < len * S5; e += 256) {
    const size_t src = (size_t)(t0 + e / S5) * a.C + h * S5 + (e % S5);
    kk[e] = a.k[src];
    vv[e] = a.v[src];
  }
  if (t < S5) wsh[t] = a.w[a.uw_head ? h : h * S5 + t];
  __syncthreads();
  float s[16];
#pragma unroll
  for (int ii = 0; ii < 16; ii++) s[ii] = 0.f;
  for (int tt = 0; tt < len; tt++) {
    const float vj = vv[tt * S5 + j];
#pragma unroll
    for (int ii = 0; ii < 16; ii++) {
      const int i = ig * 16 + ii;
      s[ii] = __builtin_fmaf(wsh[i], s[ii], kk[tt * S5 + i] * vj);
    }
  }
  float* dst = a.loc + ((size_t)ch * a.H + h) * S5 * S5;
#pragma unroll
  for (int ii = 0; ii < 16; ii++) dst[(ig * 16 + ii) * S5 + j] = s[ii];
}

// The serial pass over the chunks, one state element per thread.  The decay of the incoming state
// over a whole chunk is one multiplication by w^Lc (formed once by repeated multiplication), and the
// chunks' local end states are read eight at a time, the next eight while these are consumed.
__global__ __launch_bounds__(256) void wkv5_carry_kernel(Wkv5Seq a) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;  // element of [H][64][64]
  const size_t per = (size_t)a.H * S5 * S5;
  if (e >= per) return;
  constexpr int PF = 8;
  const int i = (int)((e / S5) % S5), h = (int)(e / (S5 * S5));
  const float w = a.w[a.uw_head ? h : h * S5 + i];
  float cur[PF], nxt[PF];
#pragma unroll
  for (int j = 0; j < PF; j++) cur[j] = a.loc[(size_t)(j < a.nchunk ? j : a.nchunk - 1) * per + e];
  float s = a.s[e];
  float wl = 1.0f;  // w^Lc; the last chunk may be shorter, but nothing is carried out of it here
  for (int q = 0; q < a.Lc; q++) wl *= w;
  for (int ch0 = 0; ch0 < a.nchunk; ch0 += PF) {
#pragma unroll
    for (int j = 0; j < PF; j++) {
      const int ch = ch0 + PF + j;
      nxt[j] = a.loc[(size_t)(ch < a.nchunk ? ch : a.nchunk - 1) * per + e];
    }
#pragma unroll
    for (int j = 0; j < PF; j++) {
      const int ch = ch0 + j;
      if (ch < a.nchunk) {
        a.sin[(size_t)ch * per + e] = s;
        s = __builtin_fmaf(wl, s, cur[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < PF; j++) cur[j] = nxt[j];
  }
}

__global__ __launch_bounds__(256) void wkv5_apply_kernel(Wkv5Seq a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* rr = reinterpret_cast<float*>(smem);  // [Lc][64]
  float* kk = rr + a.Lc * S5;
  float* vv = kk + a.Lc * S5;
  __shared__ float wsh[S5], ush[S5];
  constexpr int kGroup = 16;  // steps whose partial sums wait in LDS for one round of group norms
  __shared__ float part[kGroup][4][S5];
  const int h = blockIdx.x, ch = blockIdx.y, t = threadIdx.x, j = t & 63, ig = t >> 6;
  const int t0 = ch * a.Lc, len = min(a.Lc, a.T - t0);
  for (int e = t; e < len * S5; e += 256) {
    const size_t src = (size_t)(t0 + e / S5) * a.C + h * S5 + (e % S5);
    rr[e] = a.r[src];
    kk[e] = a.k[src];
    vv[e] = a.v[src];
  }
  if (t < S5) {
    wsh[t] = a.w[a.uw_head ? h : h * S5 + t];
    ush[t] = a.u[a.uw_head ? h : h * S5 + t];
  }
  const float* src = a.sin + ((size_t)ch * a.H + h) * S5 * S5;
  float s[16];
#pragma unroll
  for (int ii = 0; ii < 16; ii++) s[ii] = src[(ig * 16 + ii) * S5 + j];
  const float gw = a.lx_w[h * S5 + j], gb = a.lx_b[h * S5 + j];
  __syncthreads();
  float wr[16], ur[16];
#pragma unroll
  for (int ii = 0; ii < 16; ii++) {
    wr[ii] = wsh[ig * 16 + ii];
    ur[ii] = ush[ig * 16 + ii];
  }
  for (int tb = 0; tb < len; tb += kGroup) {
    const int n = min(kGroup, len - tb);
    for (int q = 0; q < n; q++) {
      const int tt = tb + q;
      const float vj = vv[tt * S5 + j];
      float acc = 0.f;
#pragma unroll
      for (int ii = 0; ii < 16; ii++) {
        const int i = ig * 16 + ii;
        const float aij = kk[tt * S5 + i] * vj;
        const float tmp = __builtin_fmaf(ur[ii], aij, s[ii]);
        s[ii] = __builtin_fmaf(wr[ii], s[ii], aij);
        acc = __builtin_fmaf(rr[tt * S5 + i], tmp, acc);
      }
      part[q][ig][j] = acc;
    }
    __syncthreads();
    // wave ig: the group norms of steps ig, ig + 4, ... of this round
    for (int q = ig; q < n; q += 4) {
      const float o = ((part[q][0][j] + part[q][1][j]) + part[q][2][j]) + part[q][3][j];
      const float mean = wave_sum(o) / (float)S5;
      const float d = o - mean;
      float var = wave_sum(d * d) / (float)S5;
      var = var > 0.f ? var : 0.f;
      const float inv = 1.0f / sqrtf(var + 1e-5f);
      const float y = d * inv * gw + gb;
      const size_t oi = (size_t)(t0 + tb + q) * a.C + h * S5 + j;
      a.gated[oi] = a.g ? (h1)y * a.g[oi] : (h1)y;
    }
    __syncthreads();  // `part` is free for the next round
  }
  if (ch == a.nchunk - 1) {
    float* dst = a.s_out + (size_t)h * S5 * S5;
#pragma unroll
    for (int ii = 0; ii < 16; ii++) dst[(ig * 16 + ii) * S5 + j] = s[ii];
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
#define FR_TRY(expr)        \
  do {                      \
    int _e = (expr);        \
    if (_e != 0) return _e; \
  } while (0)

static size_t al256(size_t n) { return (n + 255) / 256 * 256; }

static int check_w(const frhip_weight* w, int K, int N, const char* what) {
  if (!w || !w->data) return set_error(FRHIP_EINVAL, what);
  if (w->dtype != FRHIP_F16 && w->dtype != FRHIP_U8) return set_error(FRHIP_EINVAL, what);
  if (w->K != K || w->N != N) return set_error(FRHIP_ESHAPE, what);
  if (w->dtype == FRHIP_U8 && (!w->mx || !w->rx || !w->my || !w->ry)) return set_error(FRHIP_EINVAL, what);
  return 0;
}

static int launch_ln_mix(int T, int C, const void* x, const void* state, const void* ln_w, const void* ln_b,
                         const void* const* mix, h1* const* out, int nmix, void* xx_last, hipStream_t st) {
  LnMixSeq a;
  a.T = T; a.C = C; a.nmix = nmix;
  a.x = (const h1*)x; a.state = (const h1*)state; a.ln_w = (const h1*)ln_w; a.ln_b = (const h1*)ln_b;
  for (int i = 0; i < nmix; i++) {
    a.mix[i] = (const h1*)mix[i];
    a.out[i] = out[i];
  }
  a.xx_last = (h1*)xx_last;
  const int nwg = (T + kLnRows - 1) / kLnRows;
  if (C % 8 == 0 && C <= 2048)
    hipLaunchKernelGGL(ln_mix_rows_kernel<1>, dim3(nwg), dim3(256), 0, st, a);
  else if (C % 8 == 0 && C <= 4096)
    hipLaunchKernelGGL(ln_mix_rows_kernel<2>, dim3(nwg), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(ln_mix_seq_kernel, dim3(T), dim3(256), 4 * (size_t)C, st, a);
  return check_launch("ln_mix_seq");
}

// chunk length for a scan of T steps when one chunk occupies `units` workgroup-sized units:
// enough chunks to fill the device (~4 units per CU), chunks of at least 16 steps (the serial pass
// over the chunks costs about 0.18 us per chunk: at T = 1024, 64 chunks of 16 beat 128 of 8)
static int pick_chunk(int T, int units) {
  int want = (4 * compute_units() + units - 1) / units;
  if (want < 1) want = 1;
  int Lc = (T + want - 1) / want;
  if (Lc < 16) Lc = 16;
  if (Lc > 64) Lc = 64;
  return Lc;
}

}  // namespace frhip

using namespace frhip;

static size_t seq_dequant_bytes(int C, int F) {
  const size_t cc = (size_t)C * C, cf = (size_t)C * F;
  const size_t att = 4 * cc, ffn = cc + cf;
  return 2 * (att > ffn ? att : ffn);
}

extern "C" size_t frhip_seq_workspace_bytes(int T, int C, int F) {
  if (T <= 0 || C <= 0 || F <= 0) return 0;
  const size_t tc = (size_t)T * C;
  // activations: 4 mixed inputs + g + gated (half), k v r y (fp32), vx [T][F] (half)
  size_t n = 6 * al256(2 * tc) + 4 * al256(4 * tc) + al256(2 * (size_t)T * F);
  // short prompts: partial sums of the products split over K (launch_gemm's few_rows scratch)
  if (T <= kFewRowsMax) n += al256(4 * kFewRowsFloats);
  // scan scratch: RWKV-4 6 x [nchunk][C] fp32 with nchunk <= T/8+1; RWKV-5 2 x [nchunk][C*64] fp32
  const size_t nchunk = (size_t)T / 8 + 1;
  n += 6 * al256(4 * nchunk * C) + 2 * al256(4 * nchunk * (size_t)C * 64);
  // binary16 expansion of the uint8 weights of one launch: the largest group is k,v,r,g or ffn r,k
  n += al256(seq_dequant_bytes(C, F));
  return n;
}

namespace {
struct SeqWs {
  h1 *m0, *m1, *m2, *m3, *g, *gated, *vx;
  float *f0, *f1, *f2, *f3;
  float* few;        // kFewRowsFloats floats when T <= kFewRowsMax, else null
  size_t few_floats;
  float* scan;
  h1* dq;  // binary16 expansion of one launch's uint8 weights
};
SeqWs carve_seq(void* ws, int T, int C, int F) {
  const size_t tc = (size_t)T * C;
  unsigned char* p = static_cast<unsigned char*>(ws);
  SeqWs w;
  h1** hs[6] = {&w.m0, &w.m1, &w.m2, &w.m3, &w.g, &w.gated};
  for (auto h : hs) {
    *h = reinterpret_cast<h1*>(p);
    p += al256(2 * tc);
  }
  float** fs[4] = {&w.f0, &w.f1, &w.f2, &w.f3};
  for (auto f : fs) {
    *f = reinterpret_cast<float*>(p);
    p += al256(4 * tc);
  }
  w.few = T <= kFewRowsMax ? reinterpret_cast<float*>(p) : nullptr;
  w.few_floats = T <= kFewRowsMax ? kFewRowsFloats : 0;
  if (w.few) p += al256(4 * kFewRowsFloats);
  w.vx = reinterpret_cast<h1*>(p);
  p += al256(2 * (size_t)T * F);
  w.scan = reinterpret_cast<float*>(p);
  const size_t nchunk = (size_t)T / 8 + 1;
  p += 6 * al256(4 * nchunk * C) + 2 * al256(4 * nchunk * (size_t)C * 64);
  w.dq = reinterpret_cast<h1*>(p);
  return w;
}
}  // namespace

// ffn_seq (kernels/cuda/ffn_seq.cu:65-109).  x [T][C]; sx [C] shift state; xx_out [C] = LN(x)[T-1].
extern "C" int frhip_ffn_seq(int T, int C, int F, const void* x, const void* sx, const void* ln_w, const void* ln_b,
                             const void* k_mix, const void* r_mix, const frhip_weight* kw, const frhip_weight* vw,
                             const frhip_weight* rw, void* x_out, void* xx_out, int post_div2, void* workspace,
                             frhip_stream s) {
  if (T <= 0) return set_error(FRHIP_ESHAPE, "ffn_seq: T must be positive");
  if (!x || !sx || !ln_w || !ln_b || !k_mix || !r_mix || !x_out || !xx_out || !workspace)
    return set_error(FRHIP_EINVAL, "ffn_seq: null pointer");
  if (C <= 0 || C % 64 != 0 || F <= 0 || F % 64 != 0) return set_error(FRHIP_ESHAPE, "ffn_seq: C and F must be multiples of 64");
  FR_TRY(check_w(kw, C, F, "ffn_seq: bad key weight"));
  FR_TRY(check_w(vw, F, C, "ffn_seq: bad value weight"));
  FR_TRY(check_w(rw, C, C, "ffn_seq: bad receptance weight"));
  hipStream_t st = static_cast<hipStream_t>(s);
  SeqWs w = carve_seq(workspace, T, C, F);
  const void* mixes[2] = {k_mix, r_mix};
  h1* outs[2] = {w.m0, w.m1};
  FR_TRY(launch_ln_mix(T, C, x, sx, ln_w, ln_b, mixes, outs, 2, xx_out, st));
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.M = T; a.K = C;
  gemm_add_seg(a, w.m1, rw, w.m2, G_SIGMOID);  // r
  gemm_add_seg(a, w.m0, kw, w.vx, G_RELU2);    // vx
  if (kw->dtype != rw->dtype) return set_error(FRHIP_EINVAL, "ffn_seq: key/receptance dtypes differ");
  FR_TRY(launch_gemm(a, kw->dtype == FRHIP_U8, st, "ffn_seq r,k", w.dq, nullptr, 0, 0, w.few, w.few_floats));
  GemmArgs b;
  memset(&b, 0, sizeof(b));
  b.M = T; b.K = F;
  b.res_x = (const h1*)x; b.res_r = w.m2; b.div2 = post_div2 ? 1 : 0;
  gemm_add_seg(b, w.vx, vw, x_out, G_FFN_OUT);
  // the four fp32 [T][C] buffers of the workspace (unused by ffn) take the partial sums of a K-split launch
  return launch_gemm(b, vw->dtype == FRHIP_U8, st, "ffn_seq v", w.dq, w.f0, (size_t)(w.f1 - w.f0), 4, w.few, w.few_floats);
}

// RWKV-4 sequence attention.  The reference has no such operator
// (kernels/default/model_forward_seq.cpp:111-112); the result is defined by T one-token steps
// of kernels/cuda/att.cu:182-217 (model_forward_seq.cpp:34-46).
extern "C" int frhip_att_seq_v4(int T, int C, const void* x, const void* sx, const float* aa, const float* bb,
                                const float* pp, const void* ln_w, const void* ln_b, const void* k_mix,
                                const void* v_mix, const void* r_mix, const float* t_decay, const float* t_first,
                                const frhip_weight* kw, const frhip_weight* vw, const frhip_weight* rw,
                                const frhip_weight* ow, void* x_out, void* xx_out, float* aa_out, float* bb_out,
                                float* pp_out, void* workspace, frhip_stream s) {
  if (T <= 0) return set_error(FRHIP_ESHAPE, "att_seq_v4: T must be positive");
  if (!x || !sx || !aa || !bb || !pp || !ln_w || !ln_b || !k_mix || !v_mix || !r_mix || !t_decay || !t_first ||
      !x_out || !xx_out || !aa_out || !bb_out || !pp_out || !workspace)
    return set_error(FRHIP_EINVAL, "att_seq_v4: null pointer");
  if (C <= 0 || C % 64 != 0) return set_error(FRHIP_ESHAPE, "att_seq_v4: C must be a multiple of 64");
  FR_TRY(check_w(kw, C, C, "att_seq_v4: bad key weight"));
  FR_TRY(check_w(vw, C, C, "att_seq_v4: bad value weight"));
  FR_TRY(check_w(rw, C, C, "att_seq_v4: bad receptance weight"));
  FR_TRY(check_w(ow, C, C, "att_seq_v4: bad output weight"));
  if (kw->dtype != vw->dtype || kw->dtype != rw->dtype) return set_error(FRHIP_EINVAL, "att_seq_v4: k/v/r dtypes differ");
  hipStream_t st = static_cast<hipStream_t>(s);
  SeqWs w = carve_seq(workspace, T, C, 64);
  const void* mixes[3] = {k_mix, v_mix, r_mix};
  h1* outs[3] = {w.m0, w.m1, w.m2};
  FR_TRY(launch_ln_mix(T, C, x, sx, ln_w, ln_b, mixes, outs, 3, xx_out, st));
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.M = T; a.K = C;
  gemm_add_seg(a, w.m0, kw, w.f0, G_STORE_F32);  // k
  gemm_add_seg(a, w.m1, vw, w.f1, G_STORE_F32);  // v
  gemm_add_seg(a, w.m2, rw, w.m3, G_SIGMOID);    // r
  FR_TRY(launch_gemm(a, kw->dtype == FRHIP_U8, st, "att_seq_v4 k,v,r", w.dq, nullptr, 0, 0, w.few, w.few_floats));

  Wkv4Seq q;
  q.T = T; q.C = C;
  q.Lc = pick_chunk(T, (C + 255) / 256);
  // FRHIP_WKV4_SERIAL_CARRY=1: the chunk start states from a serial pass of their own (same bits)
  static const bool force_serial = getenv("FRHIP_WKV4_SERIAL_CARRY") != nullptr;
  // Without the serial pass a chunk composes the local states of all chunks before it, nchunk / 2 compositions
  // on average against Lc steps of its own: quadratic in T.  Beyond kComposeMaxChunks chunks of 32 steps
  // (T > 4096) the serial pass takes over.
  constexpr int kComposeMaxChunks = 128;
  const bool serial_carry = force_serial || (T + 31) / 32 > kComposeMaxChunks;
  // half as many, twice as long chunks (32 of 32 steps at T = 1024) cost the scans less than they save
  // the composition
  if (!serial_carry && q.Lc < 32 && T >= 512) q.Lc = 32;
  q.nchunk = (T + q.Lc - 1) / q.Lc;
  q.k = w.f0; q.v = w.f1; q.u = t_first; q.w = t_decay; q.r = w.m3;
  q.aa = aa; q.bb = bb; q.pp = pp;
  const size_t n = al256(4 * (size_t)q.nchunk * C) / 4;
  q.la = w.scan; q.lb = q.la + n; q.lp = q.lb + n; q.sa = q.lp + n; q.sb = q.sa + n; q.sp = q.sb + n;
  q.aa_out = aa_out; q.bb_out = bb_out; q.pp_out = pp_out;
  dim3 grid((C + 255) / 256, q.nchunk);
  hipLaunchKernelGGL(wkv4_local_kernel, grid, dim3(256), 0, st, q);
  if (serial_carry) {
    hipLaunchKernelGGL(wkv4_carry_kernel, dim3((C + 63) / 64), dim3(64), 0, st, q);
    hipLaunchKernelGGL(wkv4_apply_kernel<false>, grid, dim3(256), 0, st, q);
  } else {
    hipLaunchKernelGGL(wkv4_apply_kernel<true>, grid, dim3(256), 0, st, q);
  }
  FR_TRY(check_launch("wkv4_seq"));

  GemmArgs b;
  memset(&b, 0, sizeof(b));
  b.M = T; b.K = C;
  b.res_x = (const h1*)x;
  gemm_add_seg(b, w.m3, ow, x_out, G_RESIDUAL);
  return launch_gemm(b, ow->dtype == FRHIP_U8, st, "att_seq_v4 out", w.dq, nullptr, 0, 0, w.few, w.few_floats);
}

// Shared by RWKV-5.0 (no gate, u and w per head) and RWKV-5.2.
static int att_seq_v5_impl(bool v50, int T, int C, int H, const void* x, const void* sx, const float* s_in,
                                  const void* ln_w, const void* ln_b, const float* lx_w, const float* lx_b,
                                  const void* k_mix, const void* v_mix, const void* r_mix, const void* g_mix,
                                  const float* t_decay, const float* t_first, const frhip_weight* kw,
                                  const frhip_weight* vw, const frhip_weight* rw, const frhip_weight* gw,
                                  const frhip_weight* ow, void* x_out, void* xx_out, float* s_out, void* workspace,
                                  frhip_stream s) {
  if (T <= 0) return set_error(FRHIP_ESHAPE, "att_seq_v5: T must be positive");
  if (!x || !sx || !s_in || !ln_w || !ln_b || !lx_w || !lx_b || !k_mix || !v_mix || !r_mix || (!v50 && !g_mix) || !t_decay ||
      !t_first || !x_out || !xx_out || !s_out || !workspace)
    return set_error(FRHIP_EINVAL, "att_seq_v5: null pointer");
  if (H <= 0 || C % H != 0 || C / H != 64) return set_error(FRHIP_ESHAPE, "att_seq_v5: head size must be 64");
  FR_TRY(check_w(kw, C, C, "att_seq_v5: bad key weight"));
  FR_TRY(check_w(vw, C, C, "att_seq_v5: bad value weight"));
  FR_TRY(check_w(rw, C, C, "att_seq_v5: bad receptance weight"));
  if (!v50) FR_TRY(check_w(gw, C, C, "att_seq_v5: bad gate weight"));
  FR_TRY(check_w(ow, C, C, "att_seq_v5: bad output weight"));
  if (kw->dtype != vw->dtype || kw->dtype != rw->dtype || (!v50 && kw->dtype != gw->dtype))
    return set_error(FRHIP_EINVAL, "att_seq_v5: k/v/r/g dtypes differ");
  hipStream_t st = static_cast<hipStream_t>(s);
  SeqWs w = carve_seq(workspace, T, C, 64);
  const void* mixes[4] = {k_mix, v_mix, r_mix, g_mix};
  h1* outs[4] = {w.m0, w.m1, w.m2, w.m3};
  FR_TRY(launch_ln_mix(T, C, x, sx, ln_w, ln_b, mixes, outs, v50 ? 3 : 4, xx_out, st));
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.M = T; a.K = C;
  gemm_add_seg(a, w.m0, kw, w.f0, G_STORE_F32);  // k
  gemm_add_seg(a, w.m1, vw, w.f1, G_STORE_F32);  // v
  gemm_add_seg(a, w.m2, rw, w.f2, G_STORE_F32);  // r
  if (!v50) gemm_add_seg(a, w.m3, gw, w.g, G_SILU);  // g
  FR_TRY(launch_gemm(a, kw->dtype == FRHIP_U8, st, "att_seq_v5 k,v,r,g", w.dq, nullptr, 0, 0, w.few, w.few_floats));

  Wkv5Seq q;
  q.T = T; q.C = C; q.H = H;
  q.uw_head = v50 ? 1 : 0;
  q.Lc = pick_chunk(T, H);
  q.nchunk = (T + q.Lc - 1) / q.Lc;
  q.r = w.f2; q.k = w.f0; q.v = w.f1; q.w = t_decay; q.u = t_first; q.lx_w = lx_w; q.lx_b = lx_b;
  q.g = v50 ? nullptr : w.g; q.s = s_in; q.s_out = s_out; q.gated = w.gated;
  const size_t per = al256(4 * (size_t)q.nchunk * C * 64) / 4;
  q.loc = w.scan;
  q.sin = q.loc + per;
  dim3 grid(H, q.nchunk);
  hipLaunchKernelGGL(wkv5_local_kernel, grid, dim3(256), 2 * sizeof(float) * q.Lc * S5, st, q);
  hipLaunchKernelGGL(wkv5_carry_kernel, dim3(((size_t)H * S5 * S5 + 255) / 256), dim3(256), 0, st, q);
  hipLaunchKernelGGL(wkv5_apply_kernel, grid, dim3(256), 3 * sizeof(float) * q.Lc * S5, st, q);
  FR_TRY(check_launch("wkv5_seq"));

  GemmArgs b;
  memset(&b, 0, sizeof(b));
  b.M = T; b.K = C;
  b.res_x = (const h1*)x;
  gemm_add_seg(b, w.gated, ow, x_out, G_RESIDUAL);
  return launch_gemm(b, ow->dtype == FRHIP_U8, st, "att_seq_v5 out", w.dq, nullptr, 0, 0, w.few, w.few_floats);
}

// att_seq_v5_2 (kernels/cuda/att_seq.cu:368-423,464-493).
extern "C" int frhip_att_seq_v5_2(int T, int C, int H, const void* x, const void* sx, const float* s_in,
                                  const void* ln_w, const void* ln_b, const float* lx_w, const float* lx_b,
                                  const void* k_mix, const void* v_mix, const void* r_mix, const void* g_mix,
                                  const float* t_decay, const float* t_first, const frhip_weight* kw,
                                  const frhip_weight* vw, const frhip_weight* rw, const frhip_weight* gw,
                                  const frhip_weight* ow, void* x_out, void* xx_out, float* s_out, void* workspace,
                                  frhip_stream s) {
  return att_seq_v5_impl(false, T, C, H, x, sx, s_in, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, g_mix, t_decay,
                         t_first, kw, vw, rw, gw, ow, x_out, xx_out, s_out, workspace, s);
}

// att_seq_v5 (RWKV-5.0): kernels/cuda/att_seq.cu:158-256,425-462.  The reference evaluates the
// recurrence in matrix form (decay powers times r k^T, att_seq.cu:181-243); here the same sums
// are taken by the chunked scan that serves RWKV-5.2, with u and w constant over a head.
extern "C" int frhip_att_seq_v5(int T, int C, int H, const void* x, const void* sx, const float* s_in,
                                const void* ln_w, const void* ln_b, const float* lx_w, const float* lx_b,
                                const void* k_mix, const void* v_mix, const void* r_mix, const float* t_decay,
                                const float* t_first, const frhip_weight* kw, const frhip_weight* vw,
                                const frhip_weight* rw, const frhip_weight* ow, void* x_out, void* xx_out,
                                float* s_out, void* workspace, frhip_stream s) {
  return att_seq_v5_impl(true, T, C, H, x, sx, s_in, ln_w, ln_b, lx_w, lx_b, k_mix, v_mix, r_mix, nullptr, t_decay,
                         t_first, kw, vw, rw, nullptr, ow, x_out, xx_out, s_out, workspace, s);
}
