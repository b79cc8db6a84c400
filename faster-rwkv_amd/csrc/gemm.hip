// Seq-mode (prefill) matrix products on the MFMA units of gfx950.
//
//   Y[T, N] = X[T, K] . W        with W held output-major, Wt[N][K]
//
// Both operands are K-contiguous, which is the layout v_mfma_f32_32x32x16_f16 wants:
// a lane's A (or B) fragment is 8 consecutive k of one row, i.e. one 16-byte load.
// Workgroup tile 128x128 (64x128 for launches that would otherwise leave CUs idle), 2x2 compute
// waves of 64x64 (2x2 MFMA tiles, 64 fp32 accumulators per lane).  Two kernels:
//   gemm_ldw_kernel  binary16 weights: a fifth wave streams the tiles global -> LDS directly
//                    through a ring of four 64-deep K steps; the compute waves never load;
//   gemm_kernel      uint8 weights: tiles go global -> registers -> LDS (rows padded by 16 bytes
//                    against bank conflicts), the loads of step k+1 issued before the MFMAs of
//                    step k, and are dequantised to binary16 on the way into LDS with the same
//                    formula as the standalone dequantisation, so the product sees exactly the
//                    dequantised matrix.
// Products are exact in fp32, accumulation is fp32 in ascending k, and the result is rounded once
// to the output type (kernels/cuda/matmul.cpp:38-42,64-68); both kernels give the same bits.
// Independent products over the same T and K share one launch ("segments"), each with
// its own X, W and fused epilogue.
#include <climits>
#include <cstring>

#include "gemm.h"

#pragma clang fp contract(off)

namespace frhip {

typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int BN = 128;
constexpr int kGemmThreads = 256;
// Fused epilogues, shared by the product kernels: acc[i][j] is the 32x32 block (i, j) of the wave's
// (BM/2) x 64 tile at rows m0 + wm*(BM/2), columns n0 + wn*64; acc[i][j][v] is
// C[row = 8*(v/4) + 4*(lane/32) + v%4][col = lane%32] of the block.
// FULL: the workgroup's tile lies inside the matrix, nothing is predicated.  (With a predicate per
// element every store becomes a branch to an out-of-line block; on the 1024 x 6144 product that
// was 11 of 59 us.)  The epilogue kind is uniform over the launch segment: one switch, and for the
// kinds that read operands all 16 of a block are requested before the first is used.
template <int BM, bool FULL>
__device__ __forceinline__ void gemm_epilogue_t(const GemmArgs& a, const GemmSeg& sg, const f16v (&acc)[BM / 64][2],
                                                int m0, int n0, int M, int N, int lane, int wm, int wn) {
  constexpr int MI = BM / 64;
  auto for_tile = [&](int i, int j, auto&& f) {
    const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int row = m0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
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
      for (int j = 0; j < 2; j++) g(i, j, acc[i][j]);
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
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = sigmoid_h((h1)c[v]); });
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
        for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = silu_h((h1)c[v]); });
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
    gemm_epilogue_t<BM, true>(a, sg, acc, m0, n0, M, N, lane, wm, wn);
  else
    gemm_epilogue_t<BM, false>(a, sg, acc, m0, n0, M, N, lane, wm, wn);
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
// for k-segment (l%8) ^ (row%8), so k-segment q of row r sits in slot q ^ (r%8) and the MFMA
// fragment reads (32 consecutive rows, one k-segment) spread over the banks without padding.
// ---------------------------------------------------------------------------
constexpr int kLdwThreads = 320;
constexpr int kLdwStages = 4;
constexpr int kLdwBK = 64;
static constexpr size_t gemm_ldw_lds_bytes(int bm) { return (size_t)kLdwStages * (bm + BN) * kLdwBK * 2; }
__device__ __forceinline__ int ldw_at(int row, int q) { return (row >> 3) * 1024 + (row & 7) * 128 + ((q ^ (row & 7)) * 16); }

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
  const int nk = K / kLdwBK;

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
      pa[b] = sg.A + (size_t)row * K + ls * 8;
    }
#pragma unroll
    for (int b = 0; b < kBInstr; b++) {
      int row = n0 + b * 8 + lr;
      row = row < N ? row : N - 1;
      pb[b] = reinterpret_cast<const h1*>(sg.B) + (size_t)row * K + ls * 8;
    }
    auto issue = [&](int step) {
      unsigned char* st = gemm_smem + (step % kLdwStages) * kStageBytes;
      const int k0 = step * kLdwBK;
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
  gemm_epilogue<BM>(a, sg, acc, m0, n0, M, N, lane, wm, wn);
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

int launch_gemm(GemmArgs& a, bool u8, hipStream_t st, const char* what, void* dq) {
  if (a.M <= 0) return 0;
  if (a.K <= 0 || a.K % 64 != 0) return set_error(FRHIP_ESHAPE, "gemm: K must be a positive multiple of 64");
  if (u8 && dq && a.M >= kDequantRows) {
    // Expanding N x K codes costs 3 bytes of traffic per weight; the uint8 kernel's in-flight dequantisation
    // costs the launch about 0.4 x 2 T FLOP per weight at the binary16 kernel's rate: from a few hundred rows
    // on, one expansion and the binary16 kernel win.
    h1* dst = static_cast<h1*>(dq);
    for (int s = 0; s < a.nseg; s++) {
      GemmSeg& g = a.seg[s];
      if (int rc = dequant_u8_async(g.B, g.mx, g.rx, g.my, g.ry, dst, a.K, g.N, st)) return rc;
      g.B = reinterpret_cast<const unsigned char*>(dst);
      dst += (size_t)g.N * a.K;
    }
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
