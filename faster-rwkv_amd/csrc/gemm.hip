// Seq-mode (prefill) matrix products on the MFMA units of gfx950.
//
//   Y[T, N] = X[T, K] . W        with W held output-major, Wt[N][K]
//
// Both operands are K-contiguous, which is the layout v_mfma_f32_32x32x16_f16 wants:
// a lane's A (or B) fragment is 8 consecutive k of one row, i.e. one 16-byte load.
// Workgroup tile 128x128 (64x128 for launches that would otherwise leave CUs idle), 2x2 compute
// waves of 64x64 (2x2 MFMA tiles, 64 fp32 accumulators per lane).  Three kernels:
//   gemm_vw_kernel   binary16 weights, launches large enough for tiles of 128 x 128 and more:
//                    tile widths are chosen per launch so that the workgroups fill the compute
//                    units in whole rounds; loader wave and LDS ring as in gemm_ldw_kernel;
//   gemm_ldw_kernel  binary16 weights: a fifth wave streams the tiles global -> LDS directly
//                    through a ring of four 64-deep K steps; the compute waves never load;
//   gemm_kernel      uint8 weights: tiles go global -> registers -> LDS (rows padded by 16 bytes
//                    against bank conflicts), the loads of step k+1 issued before the MFMAs of
//                    step k, and are dequantised to binary16 on the way into LDS with the same
//                    formula as the standalone dequantisation, so the product sees exactly the
//                    dequantised matrix.
// Products are exact in fp32, accumulation is fp32 in ascending k, and the result is rounded once
// to the output type (kernels/cuda/matmul.cpp:38-42,64-68); all kernels give the same bits, except
// that a launch split over K (launch_gemm) adds its slices' fp32 sums at the end.
// Independent products over the same T and K share one launch ("segments"), each with
// its own X, W and fused epilogue.
#include <climits>
#include <cstring>

#include "gemm.h"

#pragma clang fp contract(off)

namespace frhip {

typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));

constexpr int BN = 128;
constexpr int kGemmThreads = 256;
// Fused epilogues, shared by the product kernels: acc[i][j] is the 32x32 block (i, j) of the wave's
// (32 MI) x (32 NJ) tile whose first element is (row0, col0); acc[i][j][v] is
// C[row = 8*(v/4) + 4*(lane/32) + v%4][col = lane%32] of the block.
// FULL: the workgroup's tile lies inside the matrix, nothing is predicated.  (With a predicate per
// element every store becomes a branch to an out-of-line block; on the 1024 x 6144 product that
// was 11 of 59 us.)  The epilogue kind is uniform over the launch segment: one switch, and for the
// kinds that read operands all 16 of a block are requested before the first is used.
// sigmoid_h of the 16 accumulators a lane holds of one 32 x 32 block, the same bits at a fraction
// of the cost.  Called element by element, sigmoid_h makes a wave take its double branch whenever
// any of its 64 lanes needs it (every other element), and its fp32 estimate alone (expf and a
// correctly rounded division, ~35 VALU instructions) is 128 x 35 instructions per lane and tile:
// the sigmoid epilogue of a 128 x 224 tile took 26 us where a plain store takes 2.5 us.
// Here the estimate is v_exp_f32 and v_rcp_f32.  Its error: t = -x log2(e) is one rounded product,
// |dt| <= 9e-8 |t|, so exp2(t) is off by at most 6.2e-8 |t| relative, which reaches the result
// scaled by e/(1+e); over the range that is not handed to the exact path anyway (x > -9.3) that
// is below 1e-6, plus one ulp each for v_exp_f32, the sum and v_rcp_f32: under 20 fp32 ulps.  An
// estimate further than 64 ulps from the midpoint of two binary16 values therefore rounds as the
// exact value does; the others (about 1 in 60) are queued per lane and evaluated in double
// afterwards, one per lane and pass.
__device__ __forceinline__ void sigmoid_h16(const f16v& c, h1 (&y)[16]) {
  h1 x[16];
  uint32_t pend = 0;
#pragma unroll
  for (int v = 0; v < 16; v++) {
    x[v] = (h1)c[v];
    const float e = __builtin_amdgcn_exp2f((float)x[v] * -1.44269504088896340736f);
    const float s32 = __builtin_amdgcn_rcpf(1.0f + e);
    const uint32_t frac = __float_as_uint(s32) & 0x1FFFu;  // the 13 fp32 mantissa bits binary16 drops
    const bool safe = s32 > 1e-4f && (frac - (0x1000u - 64u)) > 128u;
    y[v] = (h1)s32;
    pend |= safe ? 0u : (1u << v);
  }
  while (pend) {
    const int v = __builtin_ctz(pend);
    pend &= pend - 1;
    h1 xv = x[0];
#pragma unroll
    for (int u = 1; u < 16; u++) xv = (v == u) ? x[u] : xv;
    const h1 r = sigmoid_h_exact(xv);
#pragma unroll
    for (int u = 0; u < 16; u++) y[u] = (v == u) ? r : y[u];
  }
}

// silu_h of a block's 16 accumulators, the same bits, built like sigmoid_h16.  silu_h rounds
// e^-x to binary16, adds 1 in binary16 and divides x by the sum in fp32.  The estimates (v_exp_f32
// for the exponential, v_rcp_f32 for the quotient: under 20 and 3 fp32 ulps off) are taken when
// they are further than 64 ulps from a binary16 rounding boundary and in the normal binary16
// range; the other elements are queued and go through silu_h itself.
__device__ __forceinline__ void silu_h16(const f16v& c, h1 (&y)[16]) {
  h1 x[16];
  uint32_t pend = 0;
  auto far_from_boundary = [](float v) {
    const uint32_t frac = __float_as_uint(v) & 0x1FFFu;
    const float m = __builtin_fabsf(v);
    return m > 1e-4f && m < 60000.f && (frac - (0x1000u - 64u)) > 128u;
  };
#pragma unroll
  for (int v = 0; v < 16; v++) {
    x[v] = (h1)c[v];
    const float xf = (float)x[v];
    const float ef = __builtin_amdgcn_exp2f(xf * -1.44269504088896340736f);
    const h1 d = (h1)1.0f + (h1)ef;
    const float qf = xf * __builtin_amdgcn_rcpf((float)d);
    const bool safe = far_from_boundary(ef) && far_from_boundary(qf);
    y[v] = (h1)qf;
    pend |= safe ? 0u : (1u << v);
  }
  while (pend) {
    const int v = __builtin_ctz(pend);
    pend &= pend - 1;
    h1 xv = x[0];
#pragma unroll
    for (int u = 1; u < 16; u++) xv = (v == u) ? x[u] : xv;
    const h1 r = silu_h(xv);
#pragma unroll
    for (int u = 0; u < 16; u++) y[u] = (v == u) ? r : y[u];
  }
}

template <int MI, int NJ, bool FULL>
__device__ __forceinline__ void gemm_epilogue_t(const GemmArgs& a, const GemmSeg& sg, const f16v (&acc)[MI][NJ],
                                                int row0, int col0, int M, int N, int lane) {
  auto for_tile = [&](int i, int j, auto&& f) {
    const int col = col0 + j * 32 + (lane & 31);
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int row = row0 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if constexpr (FULL)
        f(v, true, (size_t)row * N + col);
      else
        f(v, row < M && col < N, (size_t)(row < M ? row : M - 1) * N + (col < N ? col : N - 1));
    }
  };
  auto for_blocks = [&](auto&& g) {
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
      for (int j = 0; j < NJ; j++) g(i, j, acc[i][j]);
  };
  switch (sg.epi) {
    case G_STORE_F16:
      for_blocks([&](int i, int j, const f16v& c) {
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = (h1)c[v]; });
      });
      break;
    case G_STORE_F32:
      for_blocks([&](int i, int j, const f16v& c) {
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<float*>(sg.out)[o] = c[v]; });
      });
      break;
    case G_SIGMOID:
      for_blocks([&](int i, int j, const f16v& c) {
        h1 y[16];
        sigmoid_h16(c, y);
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = y[v]; });
      });
      break;
    case G_RELU2:
      for_blocks([&](int i, int j, const f16v& c) {
        for_tile(i, j, [&](int v, bool ok, size_t o) {
          const h1 t = (h1)c[v];
          if (ok) static_cast<h1*>(sg.out)[o] = (t > (h1)0.0f) ? (t * t) : (h1)0.0f;
        });
      });
      break;
    case G_SILU:
      for_blocks([&](int i, int j, const f16v& c) {
        h1 y[16];
        silu_h16(c, y);
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = y[v]; });
      });
      break;
    case G_RESIDUAL:
      for_blocks([&](int i, int j, const f16v& c) {
        h1 rx[16];
        for_tile(i, j, [&](int v, bool, size_t o) { rx[v] = a.res_x[o]; });
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = rx[v] + (h1)c[v]; });
      });
      break;
    case G_FFN_OUT:
      for_blocks([&](int i, int j, const f16v& c) {
        h1 rx[16], rr[16];
        for_tile(i, j, [&](int v, bool, size_t o) {
          rx[v] = a.res_x[o];
          rr[v] = a.res_r[o];
        });
        for_tile(i, j, [&](int v, bool ok, size_t o) {
          h1 r = __builtin_fmaf16((h1)c[v], rr[v], rx[v]);
          if (a.div2) r = r / (h1)2.0f;
          if (ok) static_cast<h1*>(sg.out)[o] = r;
        });
      });
      break;
    default: break;
  }
}

template <int BM>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, const GemmSeg& sg, const f16v (&acc)[BM / 64][2], int m0,
                                              int n0, int M, int N, int lane, int wm, int wn) {
  if (m0 + BM <= M && n0 + BN <= N)
    gemm_epilogue_t<BM / 64, 2, true>(a, sg, acc, m0 + wm * (BM / 2), n0 + wn * 64, M, N, lane);
  else
    gemm_epilogue_t<BM / 64, 2, false>(a, sg, acc, m0 + wm * (BM / 2), n0 + wn * 64, M, N, lane);
}

// BM = 128 (waves 2 x 2 of 64 x 64) or 64 (waves of 32 x 64), for launches that would otherwise
// leave compute units idle.  BK = 64, or 128 for launches with about one workgroup per CU: with a
// single wave per SIMD nothing hides the round trip of the next tile's loads, so a K step lasts
// about one memory latency whatever its depth, and a deeper step halves their number.
template <int BM, int BK, bool U8>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmArgs a) {
  constexpr int LDSK = BK + 8;
  constexpr int MI = BM / 64;                      // 32-row MFMA blocks per wave
  constexpr int CPR = BK / 8;                      // 16-byte chunks of 8 halves per tile row
  constexpr int AC = BM * CPR / kGemmThreads;      // chunks of the A tile per thread
  constexpr int BC = BN * CPR / kGemmThreads;      // chunks of a binary16 B tile per thread
  constexpr int QPR = BK / 16;                     // 16-code chunks per tile row (uint8)
  constexpr int QC = BN * QPR / kGemmThreads;      // chunks of a uint8 B tile per thread
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];  // gemm_lds_bytes(BM, BK)
  h1* const As = reinterpret_cast<h1*>(gemm_smem);  // [BM][LDSK]
  h1* const Bs = As + BM * LDSK;                    // [BN][LDSK]

  // which segment does this N-tile belong to
  int sidx = 0;
#pragma unroll
  for (int i = 1; i < kGemmMaxSeg; i++) sidx += (i < a.nseg && (int)blockIdx.x >= a.tile_start[i]) ? 1 : 0;
  const GemmSeg& sg = a.seg[sidx];
  const int n0 = ((int)blockIdx.x - a.tile_start[sidx]) * BN;
  const int m0 = blockIdx.y * BM;
  const int M = a.M, K = a.K, N = sg.N;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging: a tile is 128 rows x 64 k.
  //   A (binary16): 1024 chunks of 8 halves, 4 per thread: chunk c -> row c/8, k (c%8)*8
  //   B binary16: same.  B uint8: 512 chunks of 16 codes, 2 per thread: row c/4, k (c%4)*16
  struct Stage {
    h8 ra[AC];
    h8 rb[U8 ? 1 : BC];
    u32x4 rq[U8 ? QC : 1];
  };
  auto load_tiles = [&](Stage& st, int k0) {
#pragma unroll
    for (int i = 0; i < AC; i++) {
      const int c = tid + i * kGemmThreads;
      int row = m0 + c / CPR;
      row = row < M ? row : M - 1;  // rows past M are computed on a copy of the last row and never stored
      st.ra[i] = *reinterpret_cast<const h8*>(sg.A + (size_t)row * K + k0 + (c % CPR) * 8);
    }
    if constexpr (!U8) {
#pragma unroll
      for (int i = 0; i < BC; i++) {
        const int c = tid + i * kGemmThreads;
        int row = n0 + c / CPR;
        row = row < N ? row : N - 1;
        st.rb[i] = __builtin_nontemporal_load(reinterpret_cast<const h8*>(sg.B + ((size_t)row * K + k0 + (c % CPR) * 8) * 2));
      }
    } else {
#pragma unroll
      for (int i = 0; i < QC; i++) {
        const int c = tid + i * kGemmThreads;
        int row = n0 + c / QPR;
        row = row < N ? row : N - 1;
        st.rq[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sg.B + (size_t)row * K + k0 + (c % QPR) * 16));
      }
    }
  };
  auto store_tiles = [&](const Stage& st, int k0) {
#pragma unroll
    for (int i = 0; i < AC; i++) {
      const int c = tid + i * kGemmThreads;
      *reinterpret_cast<h8*>(&As[(c / CPR) * LDSK + (c % CPR) * 8]) = st.ra[i];
    }
    if constexpr (!U8) {
#pragma unroll
      for (int i = 0; i < BC; i++) {
        const int c = tid + i * kGemmThreads;
        *reinterpret_cast<h8*>(&Bs[(c / CPR) * LDSK + (c % CPR) * 8]) = st.rb[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < QC; i++) {
        const int c = tid + i * kGemmThreads;
        int row = n0 + c / QPR;
        row = row < N ? row : N - 1;
        const int kk = k0 + (c % QPR) * 16;
        const float c2 = dequant_c(sg.rx[row]);
        const float m2 = (float)sg.mx[row];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
          const h8 ry = *reinterpret_cast<const h8*>(sg.ry + kk + hh * 8);
          const h8 my = *reinterpret_cast<const h8*>(sg.my + kk + hh * 8);
          const uint32_t w0 = st.rq[i][2 * hh], w1 = st.rq[i][2 * hh + 1];
          h2 p0 = dequant_pair<0>(w0, c2, m2, ry.s01, my.s01);
          h2 p1 = dequant_pair<1>(w0, c2, m2, ry.s23, my.s23);
          h2 p2 = dequant_pair<0>(w1, c2, m2, ry.s45, my.s45);
          h2 p3 = dequant_pair<1>(w1, c2, m2, ry.s67, my.s67);
          h8 o = {p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
          *reinterpret_cast<h8*>(&Bs[(c / QPR) * LDSK + (c % QPR) * 16 + hh * 8]) = o;
        }
      }
    }
  };

  f16v acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // the fragments of FG * 16 k are requested from LDS together; the MFMAs then start as the first
  // ones arrive instead of paying the LDS latency once per 16-deep sub-step
  auto compute_tile = [&]() {
    constexpr int FG = 4;
#pragma unroll
    for (int kh = 0; kh < BK; kh += FG * 16) {
      h8 fa[FG][MI], fb[FG][2];
#pragma unroll
      for (int kq = 0; kq < FG; kq++) {
        const int kofs = kh + kq * 16 + (lane >> 5) * 8;
#pragma unroll
        for (int i = 0; i < MI; i++)
          fa[kq][i] = *reinterpret_cast<const h8*>(&As[(wm * (BM / 2) + i * 32 + (lane & 31)) * LDSK + kofs]);
#pragma unroll
        for (int j = 0; j < 2; j++)
          fb[kq][j] = *reinterpret_cast<const h8*>(&Bs[(wn * 64 + j * 32 + (lane & 31)) * LDSK + kofs]);
      }
#pragma unroll
      for (int kq = 0; kq < FG; kq++)
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kq][i], fb[kq][j], acc[i][j], 0, 0, 0);
    }
  };

  Stage s0;
  load_tiles(s0, 0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();  // everyone is done reading the previous tile
    store_tiles(s0, k0);
    __syncthreads();
    if (k0 + BK < K) load_tiles(s0, k0 + BK);
    compute_tile();
  }

  gemm_epilogue<BM>(a, sg, acc, m0, n0, M, N, lane, wm, wn);
}

// ---------------------------------------------------------------------------
// binary16 weights: four MFMA waves and a fifth that only moves data.
//
// A compute unit keeps about 64 KB of loads in flight, and a wave that asks for more stands at its
// load instruction with everything behind it, MFMAs included.  In gemm_kernel the waves that
// compute also load, so requests are outstanding only between "issue" and "store to LDS".  Here
// wave 4 streams tiles global -> LDS directly (global_load_lds_dwordx4, no registers) into a ring
// of kLdwStages K-steps of 64 and is the only wave that ever waits for memory: two steps (64 KB
// for a 128 x 128 tile) are in flight all the time, and the MFMA waves meet it at one barrier
// per step.  Same products in the same order as gemm_kernel: the results are bit-identical.
//
// LDS layout.  One load instruction brings 8 rows x 64 k = 8 x 128 contiguous bytes (fully
// coalesced) and lands as 1 KB in lane order: lane l = row l/8, 16-byte slot l%8.  The lane asks
// for k-segment (l%8) ^ (row%8) ^ (row/8 % 2), so k-segment q of row r sits in slot
// q ^ (r%8) ^ (r/8 % 2).  A fragment read (32 consecutive rows, one k-segment) is served 16 lanes
// per cycle over 64 banks; rows r and r+8 lie 1 KB apart, i.e. on the same banks, and the last
// term moves them one slot apart: SQ_LDS_BANK_CONFLICT is 0 and a read takes 4 cycles (without
// that term every read was a two-way conflict: 8 cycles).
// ---------------------------------------------------------------------------
// global_load_lds_dwordx4 with the address as a scalar base plus a 32-bit lane offset.  The builtin
// takes a 64-bit address per lane, which costs the loader one vector add per load; on the SIMD it
// shares with an MFMA wave each of those waits for a gap between that wave's MFMAs, and the whole
// workgroup waits for the loader at the step's barrier (per K-step of a 128 x 256 tile: loader 2150
// cycles from barrier to barrier, MFMA waves 1550-1700 plus 540-700 waiting).  In this form a load
// needs scalar instructions only.  `lds` is the destination's LDS byte address (lane l writes 16 bytes
// at lds + 16 l); the wait counts are the caller's business, as with the builtin.
// M0 is written here without the compiler knowing (it refuses m0 in a clobber list: a reserved register).  That is safe
// as used: a workgroup issues either these loads or the builtin's (a tile lies wholly inside the matrices or it does not),
// never both, so no value the compiler keeps in M0 for the builtin is ever live across this statement.
__device__ __forceinline__ void load_lds_saddr(unsigned voff, const void* sbase, unsigned lds) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds) : "memory");
}

// The same address for every lane, in scalar registers (the compiler cannot always prove it).
__device__ __forceinline__ const unsigned char* uniform_ptr(const void* p) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<const unsigned char*>(((unsigned long long)hi << 32) | lo);
}

constexpr int kLdwThreads = 320;
constexpr int kLdwStages = 4;
constexpr int kLdwBK = 64;
static constexpr size_t gemm_ldw_lds_bytes(int bm) { return (size_t)kLdwStages * (bm + BN) * kLdwBK * 2; }
__device__ __forceinline__ int ldw_at(int row, int q) {
  return (row >> 3) * 1024 + (row & 7) * 128 + ((q ^ (row & 7) ^ ((row >> 3) & 1)) * 16);
}

template <int BM>
__global__ __launch_bounds__(kLdwThreads) void gemm_ldw_kernel(GemmArgs a) {
  constexpr int MI = BM / 64;
  constexpr int kABytes = BM * kLdwBK * 2, kBBytes = BN * kLdwBK * 2, kStageBytes = kABytes + kBBytes;
  constexpr int kAInstr = kABytes / 1024, kBInstr = kBBytes / 1024, kPer = kAInstr + kBInstr;
  static_assert(kPer == 32 || kPer == 24, "wait counts below are written for these");
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];

  int sidx = 0;
#pragma unroll
  for (int i = 1; i < kGemmMaxSeg; i++) sidx += (i < a.nseg && (int)blockIdx.x >= a.tile_start[i]) ? 1 : 0;
  const GemmSeg& sg = a.seg[sidx];
  const int n0 = ((int)blockIdx.x - a.tile_start[sidx]) * BN;
  const int m0 = blockIdx.y * BM;
  const int M = a.M, K = a.K, N = sg.N;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // slice z of ksplit takes K-steps [z base + min(z, rem), ...): the first rem slices one step more
  const int ksplit = a.ksplit > 1 ? a.ksplit : 1;
  const int kz = blockIdx.z, ksteps = K / kLdwBK, kper = ksteps / ksplit, krem = ksteps % ksplit;
  const int nk = kper + (kz < krem ? 1 : 0);            // K-steps of this slice
  const int kbase = (kz * kper + (kz < krem ? kz : krem)) * kLdwBK;

  if (wave == 4) {
    // ---- the loader ----
    const int lr = lane >> 3, ls = (lane & 7) ^ lr;
    // per-instruction row pointers; rows past M (N) repeat the last row and are never stored
    const h1* pa[kAInstr];
    const h1* pb[kBInstr];
#pragma unroll
    for (int b = 0; b < kAInstr; b++) {
      int row = m0 + b * 8 + lr;
      row = row < M ? row : M - 1;
      pa[b] = sg.A + (size_t)row * K + kbase + (ls ^ (b & 1)) * 8;
    }
#pragma unroll
    for (int b = 0; b < kBInstr; b++) {
      int row = n0 + b * 8 + lr;
      row = row < N ? row : N - 1;
      pb[b] = reinterpret_cast<const h1*>(sg.B) + (size_t)row * K + kbase + (ls ^ (b & 1)) * 8;
    }
    // a tile wholly inside the matrices: scalar base per load plus one of two lane offsets (load_lds_saddr)
    const bool full = m0 + BM <= M && n0 + BN <= N && (size_t)K * 16 + 128 < 0xffffffffull;
    const unsigned voff[2] = {(unsigned)(lr * K * 2 + ls * 16), (unsigned)(lr * K * 2 + (ls ^ 1) * 16)};
    const unsigned char* abase = uniform_ptr(reinterpret_cast<const unsigned char*>(sg.A) + ((size_t)m0 * K + kbase) * 2);
    const unsigned char* bbase = uniform_ptr(reinterpret_cast<const unsigned char*>(sg.B) + ((size_t)n0 * K + kbase) * 2);
    const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)gemm_smem);
    const size_t group = (size_t)__builtin_amdgcn_readfirstlane(K) * 16;
    auto issue = [&](int step) {
      const int k0 = step * kLdwBK;
      if (full) {
        const unsigned stl = lds0 + (step % kLdwStages) * kStageBytes;
        const unsigned char* ak = abase + (size_t)k0 * 2;
        const unsigned char* bk = bbase + (size_t)k0 * 2;
#pragma unroll
        for (int b = 0; b < kAInstr; b++) load_lds_saddr(voff[b & 1], ak + b * group, stl + b * 1024);
#pragma unroll
        for (int b = 0; b < kBInstr; b++) load_lds_saddr(voff[b & 1], bk + b * group, stl + kABytes + b * 1024);
        return;
      }
      unsigned char* st = gemm_smem + (step % kLdwStages) * kStageBytes;
#pragma unroll
      for (int b = 0; b < kAInstr; b++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(pa[b] + k0),
                                         (__attribute__((address_space(3))) void*)(st + b * 1024), 16, 0, 0);
#pragma unroll
      for (int b = 0; b < kBInstr; b++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(pb[b] + k0),
                                         (__attribute__((address_space(3))) void*)(st + kABytes + b * 1024), 16, 0, 0);
    };
    issue(0);
    if (nk > 1) issue(1);
    for (int k = 0; k < nk; k++) {
      // step k has landed when at most the loads of step k+1 are outstanding (loads complete in order)
      if (k + 1 < nk) {
        if constexpr (kPer == 32)
          __builtin_amdgcn_s_waitcnt(0x8F70);  // vmcnt(32)
        else
          __builtin_amdgcn_s_waitcnt(0x4F78);  // vmcnt(24)
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0)
      }
      __builtin_amdgcn_s_barrier();            // barrier k: step k may be read, step k-1 has been read by all
      if (k + 2 < nk) issue(k + 2);            // into the slot of step k-2
    }
    return;
  }

  // ---- the four MFMA waves: one barrier per step, matching the loader's ----
  const int wm = wave >> 1, wn = wave & 1;
  f16v acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
  for (int k = 0; k < nk; k++) {
    __builtin_amdgcn_s_barrier();
    const unsigned char* st = gemm_smem + (k % kLdwStages) * kStageBytes;
    h8 fa[4][MI], fb[4][2];
#pragma unroll
    for (int kb = 0; kb < 4; kb++) {
      const int q = kb * 2 + (lane >> 5);
#pragma unroll
      for (int i = 0; i < MI; i++)
        fa[kb][i] = *reinterpret_cast<const h8*>(st + ldw_at(wm * (BM / 2) + i * 32 + (lane & 31), q));
#pragma unroll
      for (int j = 0; j < 2; j++)
        fb[kb][j] = *reinterpret_cast<const h8*>(st + kABytes + ldw_at(wn * 64 + j * 32 + (lane & 31), q));
    }
#pragma unroll
    for (int kb = 0; kb < 4; kb++)
#pragma unroll
      for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kb][i], fb[kb][j], acc[i][j], 0, 0, 0);
  }
  if (a.ksplit > 1) {
    GemmSeg sp = sg;  // this slice's sums go out as fp32; the epilogue proper follows in gemm_splitk_reduce_kernel
    sp.out = a.partial + (size_t)blockIdx.z * a.partial_stride + a.part_off[sidx];
    sp.epi = G_STORE_F32;
    gemm_epilogue<BM>(a, sp, acc, m0, n0, M, N, lane, wm, wn);
  } else {
    gemm_epilogue<BM>(a, sg, acc, m0, n0, M, N, lane, wm, wn);
  }
}

// Adds the K slices of a split launch in slice order and applies each product's epilogue; a thread
// takes W consecutive outputs of a row: 16, the unit the batched sigmoid / silu work on, when one of
// the epilogues is one of those, else 8 (N % 16 == 0 either way).
// og: the thread's place within a slice, over all segments; o: within its segment's [M][N]
template <int W>
__device__ __forceinline__ void splitk_reduce_body(const GemmArgs& a, const GemmSeg& sg, size_t og, size_t o) {
  constexpr int Q = W / 4;
  float acc[W];
#pragma unroll
  for (int q = 0; q < Q; q++) {
    const f4v p = *reinterpret_cast<const f4v*>(a.partial + og + 4 * q);
#pragma unroll
    for (int i = 0; i < 4; i++) acc[4 * q + i] = p[i];
  }
  // many slices (a short prompt's launch): four are requested together and then added in slice order
  if (a.ksplit <= 4) {
    for (int z = 1; z < a.ksplit; z++) {
      const float* pz = a.partial + (size_t)z * a.partial_stride + og;
#pragma unroll
      for (int q = 0; q < Q; q++) {
        const f4v p = *reinterpret_cast<const f4v*>(pz + 4 * q);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[4 * q + i] += p[i];
      }
    }
  } else
  for (int z0 = 1; z0 < a.ksplit; z0 += 4) {
    f4v p[4][Q];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (z0 + j < a.ksplit) {
        const float* pz = a.partial + (size_t)(z0 + j) * a.partial_stride + og;
#pragma unroll
        for (int q = 0; q < Q; q++) p[j][q] = *reinterpret_cast<const f4v*>(pz + 4 * q);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (z0 + j < a.ksplit)
#pragma unroll
        for (int q = 0; q < Q; q++)
#pragma unroll
          for (int i = 0; i < 4; i++) acc[4 * q + i] += p[j][q][i];
  }
  if (sg.epi == G_STORE_F32) {
    float* out = static_cast<float*>(sg.out) + o;
#pragma unroll
    for (int q = 0; q < Q; q++) {
      f4v v;
#pragma unroll
      for (int i = 0; i < 4; i++) v[i] = acc[4 * q + i];
      *reinterpret_cast<f4v*>(out + 4 * q) = v;
    }
    return;
  }
  h1 y[W];
  switch (sg.epi) {
    case G_STORE_F16:
#pragma unroll
      for (int i = 0; i < W; i++) y[i] = (h1)acc[i];
      break;
    case G_SIGMOID:
    case G_SILU:
      if constexpr (W == 16) {
        f16v c;
#pragma unroll
        for (int i = 0; i < 16; i++) c[i] = acc[i];
        if (sg.epi == G_SIGMOID) sigmoid_h16(c, y); else silu_h16(c, y);
      }
      break;
    case G_RELU2:
#pragma unroll
      for (int i = 0; i < W; i++) {
        const h1 t = (h1)acc[i];
        y[i] = (t > (h1)0.0f) ? (t * t) : (h1)0.0f;
      }
      break;
    case G_RESIDUAL:
#pragma unroll
      for (int g = 0; g < W / 8; g++) {
        const h8 x = *reinterpret_cast<const h8*>(a.res_x + o + 8 * g);
#pragma unroll
        for (int i = 0; i < 8; i++) y[8 * g + i] = x[i] + (h1)acc[8 * g + i];
      }
      break;
    default:  // G_FFN_OUT
#pragma unroll
      for (int g = 0; g < W / 8; g++) {
        const h8 x = *reinterpret_cast<const h8*>(a.res_x + o + 8 * g), r = *reinterpret_cast<const h8*>(a.res_r + o + 8 * g);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          h1 v = __builtin_fmaf16((h1)acc[8 * g + i], r[i], x[i]);
          if (a.div2) v = v / (h1)2.0f;
          y[8 * g + i] = v;
        }
      }
      break;
  }
#pragma unroll
  for (int g = 0; g < W / 8; g++) {
    h8 v;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = y[8 * g + i];
    *reinterpret_cast<h8*>(static_cast<h1*>(sg.out) + o + 8 * g) = v;
  }
}

template <int W>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmArgs a) {
  const size_t og = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (a.nseg == 1) {  // the segment's description stays in scalar registers
    if (og < a.part_off[1]) splitk_reduce_body<W>(a, a.seg[0], og, og);
    return;
  }
  if (og >= a.part_off[a.nseg]) return;
  int sidx = 0;
#pragma unroll
  for (int i = 1; i < kGemmMaxSeg; i++) sidx += (i < a.nseg && og >= a.part_off[i]) ? 1 : 0;
  splitk_reduce_body<W>(a, a.seg[sidx], og, og - a.part_off[sidx]);
}

// Small reductions go out in workgroups of one wave, so that they spread over the compute units.
static void launch_splitk_reduce(hipStream_t st, const GemmArgs& a) {
  bool wide = false;
  for (int i = 0; i < a.nseg; i++) wide = wide || a.seg[i].epi == G_SIGMOID || a.seg[i].epi == G_SILU;
  const size_t threads = (a.part_off[a.nseg] + (wide ? 15 : 7)) / (wide ? 16 : 8);
  const unsigned block = threads >= 65536 ? 256 : 64;
  const dim3 grid((unsigned)((threads + block - 1) / block));
  if (wide)
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<16>, grid, dim3(block), 0, st, a);
  else
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel<8>, grid, dim3(block), 0, st, a);
}

template <int BM>
static void gemm_ldw_launch(dim3 grid, hipStream_t st, const GemmArgs& a) {
  constexpr size_t lds = gemm_ldw_lds_bytes(BM);
  static bool raised = false;
  if (!raised) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_ldw_kernel<BM>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = true;
  }
  hipLaunchKernelGGL((gemm_ldw_kernel<BM>), grid, dim3(kLdwThreads), lds, st, a);
}

// ---------------------------------------------------------------------------
// binary16 weights, tiles of 128 (or 256) rows and a width chosen per launch.
//
// A launch of 128 x 128 tiles over T = 1024 rows rarely comes out as a whole number of rounds over
// the compute units (k,v,r of a 2048-wide model: 384 tiles on 256 CUs take as long as 512), and a
// wider tile moves fewer bytes per product.  Here the host cuts every segment of a launch into
// tiles of 128 rows x (32 w) columns, w = base or base + 1 per segment, so that the launch has as
// many workgroups as the part has compute units (or twice, three times as many), and no tile
// straddles two segments.  The two wave columns of a workgroup take ceil(w/2) and floor(w/2)
// 32-column blocks; the loops are instantiated per block count, so the products are the same
// MFMAs in the same k order as in the other kernels and the results are bit-identical.  Loader
// wave, LDS ring (three or four K-steps of 64, whatever fits 160 KB at the launch's widest tile)
// and swizzle are those of gemm_ldw_kernel.  gemm_vw_kernel<256> has eight MFMA waves (4 x 2 of
// 64 rows each) over tiles of 256 rows and at most 160 columns; the host takes it where it saves
// a round (1024 x 2048 x 10240 as one segment: 58 us against 71 us in two rounds of 128-row tiles).
// Its predicated epilogue (edge tiles) spills a few registers; the main loop does not.
// ---------------------------------------------------------------------------
constexpr int kVwMaxW = 8;

template <int BM, int W>
__device__ __forceinline__ void vw_loader(const GemmSeg& sg, unsigned char* smem, int stage_bytes, int ns, int m0, int n0,
                                          int M, int N, int K, int lane) {
  constexpr int kVwABytes = BM * kLdwBK * 2;
  constexpr int kAInstr = kVwABytes / 1024, kBInstr = 4 * W, kPer = (kAInstr + kBInstr) <= 63 ? (kAInstr + kBInstr) : 0;
  if constexpr (kPer == 0) return;  // wider than the wait counter allows: the host never plans such a tile

  const int lr = lane >> 3, ls = (lane & 7) ^ lr;
  const h1* pa[kAInstr];
  const h1* pb[kBInstr];
#pragma unroll
  for (int b = 0; b < kAInstr; b++) {
    int row = m0 + b * 8 + lr;
    row = row < M ? row : M - 1;
    pa[b] = sg.A + (size_t)row * K + (ls ^ (b & 1)) * 8;
  }
#pragma unroll
  for (int b = 0; b < kBInstr; b++) {
    int row = n0 + b * 8 + lr;
    row = row < N ? row : N - 1;
    pb[b] = reinterpret_cast<const h1*>(sg.B) + (size_t)row * K + (ls ^ (b & 1)) * 8;
  }
  const int nk = K / kLdwBK;
  // a tile that lies wholly inside the matrices: rows are 8 K halves apart for every lane, so the address of
  // load b is a uniform base (row group b, this step's k) plus one of two lane offsets
  const bool full = m0 + BM <= M && n0 + W * 32 <= N && (size_t)K * 16 + 128 < 0xffffffffull;
  const unsigned voff[2] = {(unsigned)(lr * K * 2 + ls * 16), (unsigned)(lr * K * 2 + (ls ^ 1) * 16)};
  const unsigned char* abase = uniform_ptr(reinterpret_cast<const unsigned char*>(sg.A) + (size_t)m0 * K * 2);
  const unsigned char* bbase = uniform_ptr(reinterpret_cast<const unsigned char*>(sg.B) + (size_t)n0 * K * 2);
  const unsigned lds0 = (unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)smem);
  const size_t group = (size_t)__builtin_amdgcn_readfirstlane(K) * 16;  // bytes between row groups of 8
  auto issue = [&](int step, int slot) {
    const int k0 = step * kLdwBK;
    if (full) {
      const unsigned st = lds0 + slot * stage_bytes;
      const unsigned char* ak = abase + (size_t)k0 * 2;
      const unsigned char* bk = bbase + (size_t)k0 * 2;
#pragma unroll
      for (int b = 0; b < kAInstr; b++) load_lds_saddr(voff[b & 1], ak + b * group, st + b * 1024);
#pragma unroll
      for (int b = 0; b < kBInstr; b++) load_lds_saddr(voff[b & 1], bk + b * group, st + kVwABytes + b * 1024);
      return;
    }
    unsigned char* st = smem + slot * stage_bytes;
#pragma unroll
    for (int b = 0; b < kAInstr; b++)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(pa[b] + k0),
                                       (__attribute__((address_space(3))) void*)(st + b * 1024), 16, 0, 0);
#pragma unroll
    for (int b = 0; b < kBInstr; b++)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(pb[b] + k0),
                                       (__attribute__((address_space(3))) void*)(st + kVwABytes + b * 1024), 16, 0, 0);
  };
  issue(0, 0);
  if (nk > 1) issue(1, 1);
  int slot = 2 % ns;
  for (int k = 0; k < nk; k++) {
    if (k + 1 < nk)
      __builtin_amdgcn_s_waitcnt(((kPer >> 4) << 14) | 0x0F70 | (kPer & 15));  // vmcnt(kPer): step k has landed
    else
      __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_s_barrier();  // step k may be read; step k-1 has been read by all
    if (k + 2 < nk) {
      issue(k + 2, slot);          // ns >= 3: not the slot of step k or k+1
      slot = slot + 1 == ns ? 0 : slot + 1;
    }
  }
}

template <int BM, int NJ>
__device__ __forceinline__ void vw_mma(const GemmArgs& a, const GemmSeg& sg, const unsigned char* smem, int stage_bytes, int ns,
                                       int brow0, int m0, int n0, int M, int N, bool full, int lane, int wm) {
  constexpr int kVwABytes = BM * kLdwBK * 2;
  f16v acc[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
  const int nk = a.K / kLdwBK;
  int slot = 0;
  for (int k = 0; k < nk; k++) {
    __builtin_amdgcn_s_barrier();
    const unsigned char* st = smem + slot * stage_bytes;
    slot = slot + 1 == ns ? 0 : slot + 1;
    // fragments of KG x 16 k are requested together; with eight MFMA waves a lane has 168
    // registers and holds two of the four k-blocks of a step at a time
    constexpr int KG = BM == 128 ? 4 : 2;
#pragma unroll
    for (int kh = 0; kh < 4; kh += KG) {
      h8 fa[KG][2], fb[KG][NJ];
#pragma unroll
      for (int kb = 0; kb < KG; kb++) {
        const int q = (kh + kb) * 2 + (lane >> 5);
#pragma unroll
        for (int i = 0; i < 2; i++) fa[kb][i] = *reinterpret_cast<const h8*>(st + ldw_at(wm * 64 + i * 32 + (lane & 31), q));
#pragma unroll
        for (int j = 0; j < NJ; j++)
          fb[kb][j] = *reinterpret_cast<const h8*>(st + kVwABytes + ldw_at(brow0 + j * 32 + (lane & 31), q));
      }
#pragma unroll
      for (int kb = 0; kb < KG; kb++)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < NJ; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[kb][i], fb[kb][j], acc[i][j], 0, 0, 0);
    }
  }
  if (full)
    gemm_epilogue_t<2, NJ, true>(a, sg, acc, m0 + wm * 64, n0 + brow0, M, N, lane);
  else
    gemm_epilogue_t<2, NJ, false>(a, sg, acc, m0 + wm * 64, n0 + brow0, M, N, lane);
}

template <int BM>
__global__ __launch_bounds__(BM * 2 + 64) void gemm_vw_kernel(GemmArgs a) {
  constexpr int kVwABytes = BM * kLdwBK * 2, kLoader = BM / 32;  // BM / 32 MFMA waves of 64 rows x half the width, then the loader
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
  // Workgroups are dealt to the eight XCDs in turn (linear index mod 8), each with an L2 of its own.
  // XCD x therefore takes the x-th eighth of the N tiles, for every strip of rows: it fetches
  // those weights once and one segment's rows of A, instead of every segment's.  (A matter of
  // traffic only: any assignment of tiles to workgroups gives the same results.)
  int bx = blockIdx.x, by = blockIdx.y;
  if (gridDim.x % 8 == 0) {
    const int lin = by * gridDim.x + bx, per = gridDim.x / 8;
    const int r = lin >> 3;
    bx = (lin & 7) * per + r % per;
    by = r / per;
  }
  int sidx = 0;
#pragma unroll
  for (int i = 1; i < kGemmMaxSeg; i++) sidx += (i < a.nseg && bx >= a.tile_start[i]) ? 1 : 0;
  const GemmSeg& sg = a.seg[sidx];
  const int ti = bx - a.tile_start[sidx];
  const int base = a.vw_base[sidx], wide = a.vw_wide[sidx];
  const int width = base + (ti < wide ? 1 : 0);                  // 32-column blocks of this tile
  const int n0 = (ti * base + (ti < wide ? ti : wide)) * 32;
  const int m0 = by * BM;
  const int M = a.M, K = a.K, N = sg.N;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int stage_bytes = kVwABytes + a.vw_maxw * 4096, ns = a.vw_ns;
  if (wave == kLoader) {
    switch (width) {
      case 2: vw_loader<BM, 2>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
      case 3: vw_loader<BM, 3>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
      case 4: vw_loader<BM, 4>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
      case 5: vw_loader<BM, 5>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
      case 6: vw_loader<BM, 6>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
      case 7: vw_loader<BM, BM == 128 ? 7 : 6>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;  // 256 rows: never wider than 5
      default: vw_loader<BM, BM == 128 ? 8 : 6>(sg, gemm_smem, stage_bytes, ns, m0, n0, M, N, K, lane); break;
    }
    return;
  }
  const int wm = wave >> 1, wn = wave & 1;
  const int nj0 = (width + 1) >> 1;
  const int nj = wn ? width - nj0 : nj0;
  const int brow0 = wn ? nj0 * 32 : 0;
  const bool full = m0 + BM <= M && n0 + width * 32 <= N;
  switch (nj) {
    case 1: vw_mma<BM, 1>(a, sg, gemm_smem, stage_bytes, ns, brow0, m0, n0, M, N, full, lane, wm); break;
    case 2: vw_mma<BM, 2>(a, sg, gemm_smem, stage_bytes, ns, brow0, m0, n0, M, N, full, lane, wm); break;
    case 3: vw_mma<BM, 3>(a, sg, gemm_smem, stage_bytes, ns, brow0, m0, n0, M, N, full, lane, wm); break;
    default: vw_mma<BM, BM == 128 ? 4 : 3>(a, sg, gemm_smem, stage_bytes, ns, brow0, m0, n0, M, N, full, lane, wm); break;
  }
}

// Cuts the launch into tiles of bm rows for gemm_vw_kernel<bm>: the fewest rounds over `cus` compute
// units whose widest tile fits.  Returns the number of rounds, or 0: the launch is too small for
// tiles of at least bm x 128 (the other kernels' 64-row tiles serve it better) or too ragged.
static int plan_vw(GemmArgs& a, int bm, int cus, dim3* grid, size_t* lds) {
  const int mt = (a.M + bm - 1) / bm;
  const int abytes = bm * kLdwBK * 2;
  const int wcap = bm == 128 ? kVwMaxW : 5;  // 256 rows: three stages of (256 + 160) x 64 halves are 156 KB of the 160 KB
  int cb[kGemmMaxSeg], total = 0;
  for (int s = 0; s < a.nseg; s++) {
    cb[s] = (a.seg[s].N + 31) / 32;
    total += cb[s];
  }
  for (int rounds = 1; rounds <= 4; rounds++) {
    const int P = rounds * cus / mt;  // tiles per strip of 128 rows
    if (P < a.nseg) continue;
    int t[kGemmMaxSeg], used = 0;
    for (int s = 0; s < a.nseg; s++) {
      t[s] = (int)((long)P * cb[s] / total);
      if (t[s] < 1) t[s] = 1;
      used += t[s];
    }
    if (used > P) continue;
    // the spare tiles go where the tiles are widest; among equals, to the segment whose epilogue
    // costs most (a transcendental per element), so that its tiles are the narrow ones
    auto heavy = [&](int s) { return a.seg[s].epi == G_SIGMOID || a.seg[s].epi == G_SILU ? 1 : 0; };
    while (used < P) {
      int best = 0;
      for (int s = 1; s < a.nseg; s++) {
        const long l = (long)cb[s] * t[best], r = (long)cb[best] * t[s];
        if (l > r || (l == r && heavy(s) > heavy(best))) best = s;
      }
      t[best]++;
      used++;
    }
    int maxw = 0, minw = INT_MAX;
    for (int s = 0; s < a.nseg; s++) {
      const int w = (cb[s] + t[s] - 1) / t[s];
      maxw = w > maxw ? w : maxw;
      minw = cb[s] / t[s] < minw ? cb[s] / t[s] : minw;
    }
    if (maxw > wcap) continue;
    if (minw < 2 || maxw < 4) return 0;
    int tiles = 0;
    for (int s = 0; s < a.nseg; s++) {
      a.tile_start[s] = tiles;
      a.vw_base[s] = cb[s] / t[s];
      a.vw_wide[s] = cb[s] % t[s];
      tiles += t[s];
    }
    for (int s = a.nseg; s <= kGemmMaxSeg; s++) a.tile_start[s] = INT_MAX;
    a.tile_start[a.nseg] = tiles;
    a.vw_maxw = maxw;
    const size_t stage = abytes + (size_t)maxw * 4096;
    a.vw_ns = stage * 4 <= 160 * 1024 ? 4 : 3;
    if (stage * a.vw_ns > 160 * 1024) return 0;
    *lds = stage * a.vw_ns;
    *grid = dim3(tiles, mt);
    return rounds;
  }
  return 0;
}

template <int BM>
static void gemm_vw_launch(dim3 grid, size_t lds, hipStream_t st, const GemmArgs& a) {
  static bool raised = false;
  if (!raised) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_vw_kernel<BM>), hipFuncAttributeMaxDynamicSharedMemorySize,
                              160 * 1024);
    raised = true;
  }
  hipLaunchKernelGGL((gemm_vw_kernel<BM>), grid, dim3(BM * 2 + 64), lds, st, a);
}

static constexpr size_t gemm_lds_bytes(int bm, int bk) { return (size_t)(bm + BN) * (bk + 8) * 2; }

// Tiles above 64 KB of LDS need the limit raised once per kernel.
template <int BM, int BK, bool U8>
static void gemm_launch_one(dim3 grid, hipStream_t st, const GemmArgs& a) {
  constexpr size_t lds = gemm_lds_bytes(BM, BK);
  static bool raised = false;
  if (lds > 64 * 1024 && !raised) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<BM, BK, U8>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    raised = true;
  }
  hipLaunchKernelGGL((gemm_kernel<BM, BK, U8>), grid, dim3(kGemmThreads), lds, st, a);
}
#define FR_GEMM_LAUNCH(BM_, BK_)                         \
  do {                                                   \
    if (u8)                                              \
      gemm_launch_one<BM_, BK_, true>(grid, st, a);      \
    else                                                 \
      gemm_launch_one<BM_, BK_, false>(grid, st, a);     \
  } while (0)

// FRHIP_GEMM_BK=64|128 forces the K-step depth (measurement aid); default: 128 where K allows
// (256 was measured no faster than 128).
static int env_bk() {
  const char* e = getenv("FRHIP_GEMM_BK");
  return e ? atoi(e) : 0;
}

int launch_gemm(GemmArgs& a, bool u8, hipStream_t st, const char* what, void* dq, float* partial, size_t partial_stride,
                int max_split, float* few_rows, size_t few_rows_floats) {
  if (a.M <= 0) return 0;
  if (a.K <= 0 || a.K % 64 != 0) return set_error(FRHIP_ESHAPE, "gemm: K must be a positive multiple of 64");
  if (u8 && dq && a.M >= kDequantRows) {
    // Expanding N x K codes costs 3 bytes of traffic per weight.  The uint8 kernel's in-flight dequantisation costs a launch
    // of many rows about 0.4 x 2 T FLOP per weight at the binary16 kernel's rate, and a launch of few rows cannot be spread
    // over the idle compute units as the binary16 one can (few_rows below): with scratch for it, one expansion and the
    // binary16 kernels win from a handful of rows on.
    h1* dst = static_cast<h1*>(dq);
    const unsigned char* qs[kGemmMaxSeg];
    const h1 *mxs[kGemmMaxSeg], *rxs[kGemmMaxSeg], *mys[kGemmMaxSeg], *rys[kGemmMaxSeg];
    h1* dsts[kGemmMaxSeg];
    int ns[kGemmMaxSeg];
    for (int s = 0; s < a.nseg; s++) {
      GemmSeg& g = a.seg[s];
      qs[s] = g.B; mxs[s] = g.mx; rxs[s] = g.rx; mys[s] = g.my; rys[s] = g.ry; ns[s] = g.N;
      dsts[s] = dst;
      g.B = reinterpret_cast<const unsigned char*>(dst);
      dst += (size_t)g.N * a.K;
    }
    if (int rc = dequant_u8_group_async(a.nseg, qs, mxs, rxs, mys, rys, dsts, a.K, ns, st)) return rc;
    u8 = false;
  }
  int tiles = 0;
  for (int s = 0; s < a.nseg; s++) {
    a.tile_start[s] = tiles;
    tiles += (a.seg[s].N + BN - 1) / BN;
  }
  for (int s = a.nseg; s <= kGemmMaxSeg; s++) a.tile_start[s] = INT_MAX;
  a.tile_start[a.nseg] = tiles;
  // 128-row tiles unless that leaves fewer than ~1.5 workgroups per CU; then 64-row tiles
  const int m128 = (a.M + 127) / 128;
  static const int force_bm = getenv("FRHIP_GEMM_BM") ? atoi(getenv("FRHIP_GEMM_BM")) : 0;  // measurement aid
  const bool small = force_bm ? force_bm == 64 : (long)tiles * m128 < (long)compute_units() * 3 / 2;
  static const int force_bk = env_bk();
  const bool deep = force_bk ? force_bk == 128 : true;
  const bool deep_ok = deep && a.K % 128 == 0;
  // binary16 weights go to the kernel with the loader wave (FRHIP_GEMM_LDW=0 selects the other one:
  // measurement aid); uint8 weights need the registers in between for the dequantisation
  static const bool ldw = !(getenv("FRHIP_GEMM_LDW") && atoi(getenv("FRHIP_GEMM_LDW")) == 0);
  // Split K: a single product with few outputs and a long K (ffn value: 1024 x 8192 x 2048) fills the compute units only
  // with 64 x 128 tiles, which ask L2 for 1.5 times the bytes of 128 x 128 tiles per product and are bound by just that
  // (786 MB in 57 us).  With scratch for the partial sums the launch runs ksplit slices of K over 128 x 128 tiles, and a
  // second kernel adds the slices in order and applies the epilogue.  The sums are grouped by slice, so the result can
  // differ from the unsplit launch in the last fp32 bit before the rounding to binary16.  FRHIP_GEMM_SPLITK=0: off.
  static const bool splitk = !(getenv("FRHIP_GEMM_SPLITK") && atoi(getenv("FRHIP_GEMM_SPLITK")) == 0);
  // Few rows (a short prompt): 64 x 128 tiles leave most compute units without a workgroup, and a workgroup pulls its
  // weights through a ring of two K-steps (48 KB in flight), so a launch takes K / 64 round trips to memory however few
  // rows there are (T = 64, 2048 x 2048: 16 workgroups, 17-25 us for 8 MB).  With scratch for the partial sums such a
  // launch is split over K into as many slices as there are idle compute units (at least four K-steps each), and the
  // reduction pass adds the slices in order and applies each product's epilogue.  A group that is too wide for that as a
  // whole goes out product by product, so that its narrow members still can.  FRHIP_GEMM_FEW_ROWS=0: off.
  static const bool few = !(getenv("FRHIP_GEMM_FEW_ROWS") && atoi(getenv("FRHIP_GEMM_FEW_ROWS")) == 0);
  if (!u8 && ldw && splitk && few && !force_bm && few_rows) {
    const int m64 = (a.M + 63) / 64, ksteps = a.K / kLdwBK, cus = compute_units();
    bool eligible = (long)tiles * m64 * 2 <= cus && ksteps >= 4;
    for (int sgi = 0; sgi < a.nseg; sgi++) eligible = eligible && a.seg[sgi].N % 16 == 0;
    if (eligible) {
      size_t cols = 0;
      for (int sgi = 0; sgi < a.nseg; sgi++) {
        a.part_off[sgi] = (size_t)a.M * cols;
        cols += (size_t)a.seg[sgi].N;
      }
      a.part_off[a.nseg] = (size_t)a.M * cols;
      const size_t stride = (a.part_off[a.nseg] + 63) / 64 * 64;
      long S = cus / ((long)tiles * m64);
      if (S > ksteps / 4) S = ksteps / 4;  // at least four K-steps per slice: twice the ring's depth in flight
      if ((size_t)S * stride > few_rows_floats) S = (long)(few_rows_floats / stride);
      if (S >= 2) {
        a.ksplit = (int)S;
        a.partial = few_rows;
        a.partial_stride = stride;
        gemm_ldw_launch<64>(dim3(tiles, m64, (unsigned)S), st, a);
        if (int rc = check_launch(what)) return rc;
        launch_splitk_reduce(st, a);
        return check_launch(what);
      }
    } else if (a.nseg > 1 && ksteps >= 4 && (long)tiles * m64 < cus) {  // a group that fills the part as it is stays one launch
      bool some = false;
      for (int sgi = 0; sgi < a.nseg; sgi++)
        some = some || ((long)((a.seg[sgi].N + BN - 1) / BN) * m64 * 2 <= cus && a.seg[sgi].N % 16 == 0);
      if (some) {
        for (int sgi = 0; sgi < a.nseg; sgi++) {
          GemmArgs one = a;
          one.nseg = 1;
          one.seg[0] = a.seg[sgi];
          if (int rc = launch_gemm(one, false, st, what, nullptr, nullptr, 0, 0, few_rows, few_rows_floats)) return rc;
        }
        return 0;
      }
    }
  }
  if (!u8 && ldw && splitk && !force_bm && partial && max_split >= 2 && a.nseg == 1 && a.K >= 4096 && a.seg[0].N % 16 == 0 &&
      (a.seg[0].epi == G_STORE_F16 || a.seg[0].epi == G_STORE_F32 || a.seg[0].epi == G_RESIDUAL || a.seg[0].epi == G_FFN_OUT) &&
      (size_t)a.M * a.seg[0].N <= partial_stride) {
    const long t128 = (long)tiles * m128;
    int S = (int)(compute_units() / t128);
    if (S > max_split) S = max_split;
    while (S >= 2 && a.K / (kLdwBK * S) < 16) S--;
    if (S >= 2 && t128 * S * 5 >= (long)compute_units() * 3) {  // the slices fill at least 60 % of the CUs
      a.ksplit = S;
      a.partial = partial;
      a.partial_stride = partial_stride;
      a.part_off[0] = 0;
      a.part_off[1] = (size_t)a.M * a.seg[0].N;
      gemm_ldw_launch<128>(dim3(tiles, m128, S), st, a);
      if (int rc = check_launch(what)) return rc;
      launch_splitk_reduce(st, a);
      return check_launch(what);
    }
  }
  // FRHIP_GEMM_VW=0 keeps binary16 launches on the fixed 128 / 64 x 128 tiles (measurement aid)
  static const bool vw = !(getenv("FRHIP_GEMM_VW") && atoi(getenv("FRHIP_GEMM_VW")) == 0);
  static const int force_vw_bm = getenv("FRHIP_GEMM_VW_BM") ? atoi(getenv("FRHIP_GEMM_VW_BM")) : 0;  // measurement aid
  if (!u8 && ldw && vw && !force_bm) {
    // 128-row tiles unless 256-row tiles (eight MFMA waves) need fewer rounds
    GemmArgs b1 = a, b2 = a;
    dim3 g1, g2;
    size_t l1 = 0, l2 = 0;
    const int r1 = plan_vw(b1, 128, compute_units(), &g1, &l1);
    const int r2 = force_vw_bm == 128 ? 0 : plan_vw(b2, 256, compute_units(), &g2, &l2);
    // A grouped launch that needs two rounds although each of its products alone fits one (ffn r,k at T = 1024:
    // 2048 columns in one round of 64 x 128 tiles, 8192 in one round of 128 x 256) goes out as separate launches.
    static const bool separate = !(getenv("FRHIP_GEMM_SEPARATE") && atoi(getenv("FRHIP_GEMM_SEPARATE")) == 0);
    if (separate && a.nseg > 1 && (r1 == 0 || r1 >= 2) && (r2 == 0 || r2 >= 2)) {
      bool each_one_round = true;
      for (int sgi = 0; sgi < a.nseg && each_one_round; sgi++) {
        GemmArgs one = a;
        one.nseg = 1;
        one.seg[0] = a.seg[sgi];
        dim3 g;
        size_t l = 0;
        const int rr1 = plan_vw(one, 128, compute_units(), &g, &l), rr2 = plan_vw(one, 256, compute_units(), &g, &l);
        const long t64 = (long)((a.seg[sgi].N + BN - 1) / BN) * ((a.M + 63) / 64);
        each_one_round = rr1 == 1 || rr2 == 1 || (rr1 == 0 && rr2 == 0 && t64 <= compute_units());
      }
      if (each_one_round) {
        for (int sgi = 0; sgi < a.nseg; sgi++) {
          GemmArgs one = a;
          one.nseg = 1;
          one.seg[0] = a.seg[sgi];
          if (int rc = launch_gemm(one, false, st, what, nullptr, nullptr, 0, 0, nullptr, 0)) return rc;
        }
        return 0;
      }
    }
    if (r2 && (!r1 || r2 < r1 || force_vw_bm == 256)) {
      gemm_vw_launch<256>(g2, l2, st, b2);
      return check_launch(what);
    }
    if (r1) {
      gemm_vw_launch<128>(g1, l1, st, b1);
      return check_launch(what);
    }
  }
  if (!u8 && ldw) {
    if (small)
      gemm_ldw_launch<64>(dim3(tiles, (a.M + 63) / 64), st, a);
    else
      gemm_ldw_launch<128>(dim3(tiles, m128), st, a);
    return check_launch(what);
  }
  if (small) {
    dim3 grid(tiles, (a.M + 63) / 64);
    if (deep_ok) FR_GEMM_LAUNCH(64, 128); else FR_GEMM_LAUNCH(64, 64);
  } else {
    dim3 grid(tiles, m128);
    if (deep_ok) FR_GEMM_LAUNCH(128, 128); else FR_GEMM_LAUNCH(128, 64);
  }
  return check_launch(what);
}

void gemm_add_seg(GemmArgs& a, const void* A, const frhip_weight* w, void* out, int epi) {
  GemmSeg& s = a.seg[a.nseg++];
  s.A = static_cast<const h1*>(A);
  s.B = static_cast<const unsigned char*>(w->data);
  s.mx = static_cast<const h1*>(w->mx);
  s.rx = static_cast<const h1*>(w->rx);
  s.my = static_cast<const h1*>(w->my);
  s.ry = static_cast<const h1*>(w->ry);
  s.out = out;
  s.N = w->N;
  s.epi = epi;
}

}  // namespace frhip

using namespace frhip;

// matmul, matrix x matrix (kernels/cuda/matmul.cpp:110-121): x [T][K] binary16, y [T][N].
extern "C" int frhip_gemm(const void* x, const frhip_weight* w, void* y, int T, int out_dtype, frhip_stream s) {
  if (!x || !w || !w->data || !y) return set_error(FRHIP_EINVAL, "gemm: null pointer");
  if (T < 0) return set_error(FRHIP_ESHAPE, "gemm: negative T");
  if (out_dtype != FRHIP_F16 && out_dtype != FRHIP_F32) return set_error(FRHIP_EINVAL, "gemm: out_dtype must be F16 or F32");
  if (w->dtype != FRHIP_F16 && w->dtype != FRHIP_U8) return set_error(FRHIP_EINVAL, "gemm: weight dtype must be F16 or U8");
  if (w->dtype == FRHIP_U8 && (!w->mx || !w->rx || !w->my || !w->ry)) return set_error(FRHIP_EINVAL, "gemm: uint8 weight without mx/rx/my/ry");
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(w->data) % 16 != 0)
    return set_error(FRHIP_EINVAL, "gemm: operands must be 16-byte aligned");
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.M = T;
  a.K = w->K;
  gemm_add_seg(a, x, w, y, out_dtype == FRHIP_F32 ? G_STORE_F32 : G_STORE_F16);
  return launch_gemm(a, w->dtype == FRHIP_U8, static_cast<hipStream_t>(s), "gemm");
}

static_assert(FRHIP_ACT_SIGMOID == G_SIGMOID && FRHIP_ACT_RELU2 == G_RELU2 && FRHIP_ACT_SILU == G_SILU, "activation codes");

// matmul + in-place activation (kernels/cuda/ffn_seq.cu:78-81, att_seq.cu:394-395) in one launch.
extern "C" int frhip_gemm_act(const void* x, const frhip_weight* w, void* y, int T, int act, frhip_stream s) {
  if (!x || !w || !w->data || !y) return set_error(FRHIP_EINVAL, "gemm_act: null pointer");
  if (T < 0) return set_error(FRHIP_ESHAPE, "gemm_act: negative T");
  if (act != FRHIP_ACT_SIGMOID && act != FRHIP_ACT_RELU2 && act != FRHIP_ACT_SILU)
    return set_error(FRHIP_EINVAL, "gemm_act: act must be SIGMOID, RELU2 or SILU");
  if (w->dtype != FRHIP_F16 && w->dtype != FRHIP_U8) return set_error(FRHIP_EINVAL, "gemm_act: weight dtype must be F16 or U8");
  if (w->dtype == FRHIP_U8 && (!w->mx || !w->rx || !w->my || !w->ry)) return set_error(FRHIP_EINVAL, "gemm_act: uint8 weight without mx/rx/my/ry");
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || reinterpret_cast<uintptr_t>(w->data) % 16 != 0)
    return set_error(FRHIP_EINVAL, "gemm_act: operands must be 16-byte aligned");
  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.M = T;
  a.K = w->K;
  gemm_add_seg(a, x, w, y, act);
  return launch_gemm(a, w->dtype == FRHIP_U8, static_cast<hipStream_t>(s), "gemm_act");
}
