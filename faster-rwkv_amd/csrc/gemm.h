// Argument structures of the MFMA GEMM shared by gemm.hip and seq.hip.
#pragma once

#include "device_utils.h"
#include "frhip_internal.h"

namespace frhip {

constexpr int kGemmMaxSeg = 4;

enum GemmEpi : int {
  G_STORE_F16 = 0,
  G_STORE_F32 = 1,
  G_SIGMOID = 2,    // half(sigmoid(half(acc)))                        ffn_seq.cu:78-79, att.cu:203
  G_RELU2 = 3,      // relu(half(acc))^2                               ffn_seq.cu:80-81
  G_SILU = 4,       // silu(half(acc))                                 att_seq.cu:394-395
  G_RESIDUAL = 5,   // x + half(acc)                                   att_seq.cu:412-415
  G_FFN_OUT = 6     // fma(half(acc), r, x) [/ 2]                      ffn_seq.cu:82-85, model_forward_seq.cpp:163-165
};

struct GemmSeg {
  const h1* A;                       // [M][K]
  const unsigned char* B;            // [N][K] binary16 or uint8
  const h1 *mx, *rx, *my, *ry;       // uint8 only
  void* out;                         // [M][N]
  int N, epi;
};

struct GemmArgs {
  int M, K, nseg;
  int tile_start[kGemmMaxSeg + 1];  // first N-tile of each segment
  size_t part_off[kGemmMaxSeg + 1]; // split launches: where each segment's [M][N] block starts within a slice of `partial` (floats); [nseg] = all
  // gemm_vw_kernel: a segment's tiles are vw_base (the first vw_wide of them vw_base + 1) blocks of 32 columns wide
  int vw_base[kGemmMaxSeg], vw_wide[kGemmMaxSeg], vw_maxw, vw_ns;
  GemmSeg seg[kGemmMaxSeg];
  // split K (single-segment launches of gemm_ldw_kernel<128> only): slice z of ksplit accumulates K / ksplit of the
  // product into partial + z * partial_stride as fp32 [M][N]; gemm_splitk_reduce_kernel adds the slices and applies the epilogue
  int ksplit;
  float* partial;
  size_t partial_stride;
  const h1* res_x;  // [M][N] G_RESIDUAL, G_FFN_OUT
  const h1* res_r;  // [M][N] G_FFN_OUT
  int div2;
};

// dq: optional scratch of gemm_dequant_bytes(a) bytes.  With it, uint8 weights of a launch with at least
// kDequantRows rows are expanded once to binary16 (the standalone dequantisation: the same bits as the
// in-kernel one) and the launch takes the binary16 kernel.
// partial: optional fp32 scratch of max_split slices of partial_stride floats (>= M * N each) for splitting K.
// few_rows: optional fp32 scratch of few_rows_floats floats; with it a launch of so few rows that 64 x 128 tiles leave
// at least half of the compute units idle goes out product by product, each split over K across the idle units.
constexpr size_t kFewRowsFloats = (size_t)512 * 64 * 128;  // two 64 x 128 tiles per compute unit of a 256-unit part
constexpr int kFewRowsMax = 360;                          // rows up to which the seq operators carry that scratch
int launch_gemm(GemmArgs& a, bool u8, hipStream_t st, const char* what, void* dq = nullptr, float* partial = nullptr,
                size_t partial_stride = 0, int max_split = 0, float* few_rows = nullptr, size_t few_rows_floats = 0);
constexpr int kDequantRows = FRHIP_SEQ_EXPAND_ROWS;
// uint8 [N][K] -> binary16 [N][K] with the frozen formula (ops.hip)
int dequant_u8_async(const unsigned char* q, const h1* mx, const h1* rx, const h1* my, const h1* ry, h1* dst, int K, int N,
                     hipStream_t st);
// the same for the nseg matrices of a grouped product (same K), one launch where the shapes allow it
int dequant_u8_group_async(int nseg, const unsigned char* const* q, const h1* const* mx, const h1* const* rx, const h1* const* my,
                           const h1* const* ry, h1* const* dst, int K, const int* N, hipStream_t st);
void gemm_add_seg(GemmArgs& a, const void* A, const frhip_weight* w, void* out, int epi);

}  // namespace frhip
