// Seq-mode (prefill) matrix products on the MFMA units of gfx950.
//
//   Y[T, N] = X[T, K] . W        with W held output-major, Wt[N][K]
//
// Both operands are K-contiguous, which is the layout v_mfma_f32_32x32x16_f16 wants:
// a lane's A (or B) fragment is 8 consecutive k of one row, i.e. one 16-byte load.
// Workgroup tile 128x128 (64x128 for launches that would otherwise leave CUs idle), K step 64 (128 for
// launches of about one workgroup per CU),
// 256 threads = 2x2 waves of 64x64 (2x2 MFMA tiles, 64 fp32 accumulators per lane).  Tiles of X and Wt go global -> registers -> LDS
// (rows padded by 16 bytes against bank conflicts); the loads of step k+1 are issued
// before the MFMAs of step k.  uint8 weights are dequantised to binary16 on their way
// into LDS with the same formula as the one-token kernels, so the product sees exactly
// the dequantised matrix.  Products are exact in fp32, accumulation is fp32, and the
// result is rounded once to the output type (kernels/cuda/matmul.cpp:38-42,64-68).
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

  // epilogue: acc[i][j][v] is C[row = 8*(v/4) + 4*(lane/32) + v%4][col = lane%32] of the 32x32 tile.
  // The epilogue kind is uniform over the launch segment: branch once, and for the kinds that read
  // operands request all 16 of a tile before the first is used.
  auto for_tile = [&](int i, int j, auto&& f) {
    const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int row = m0 + wm * (BM / 2) + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      f(v, row < M && col < N, (size_t)(row < M ? row : M - 1) * N + (col < N ? col : N - 1));
    }
  };
#pragma unroll
  for (int i = 0; i < MI; i++) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const f16v& c = acc[i][j];
      switch (sg.epi) {
        case G_STORE_F16:
          for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = (h1)c[v]; });
          break;
        case G_STORE_F32:
          for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<float*>(sg.out)[o] = c[v]; });
          break;
        case G_SIGMOID:
          for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = sigmoid_h((h1)c[v]); });
          break;
        case G_RELU2:
          for_tile(i, j, [&](int v, bool ok, size_t o) {
            const h1 t = (h1)c[v];
            if (ok) static_cast<h1*>(sg.out)[o] = (t > (h1)0.0f) ? (t * t) : (h1)0.0f;
          });
          break;
        case G_SILU:
          for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = silu_h((h1)c[v]); });
          break;
        case G_RESIDUAL: {
          h1 rx[16];
          for_tile(i, j, [&](int v, bool, size_t o) { rx[v] = a.res_x[o]; });
          for_tile(i, j, [&](int v, bool ok, size_t o) { if (ok) static_cast<h1*>(sg.out)[o] = rx[v] + (h1)c[v]; });
          break;
        }
        case G_FFN_OUT: {
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
          break;
        }
        default: break;
      }
    }
  }
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

int launch_gemm(GemmArgs& a, bool u8, hipStream_t st, const char* what) {
  if (a.M <= 0) return 0;
  if (a.K <= 0 || a.K % 64 != 0) return set_error(FRHIP_ESHAPE, "gemm: K must be a positive multiple of 64");
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
