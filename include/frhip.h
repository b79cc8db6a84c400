/*
 * frhip.h -- C ABI of the MI355X (gfx950) RWKV inference kernels.
 *
 * This is the boundary a faster-rwkv `hip` device binds to: the host-side operator
 * functions registered in kernels/registry.h for Device::kHIP call nothing but these
 * entry points.  Plain pointers and sizes only; no C++ or HIP types cross it.
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t value when the HIP
 *     runtime failed, or a negative FRHIP_E* value when the arguments are rejected
 *     before anything is launched.  Nothing throws.  frhip_error_string() describes
 *     the most recent failure of the calling thread.
 *   - `stream` is an opaque handle from frhip_stream_create(), or NULL for the
 *     default (null) stream.  All launches are asynchronous with respect to the host.
 *   - device pointers are plain `void *`; binary16 data is IEEE half, "f32" is float.
 *   - activations are vectors [C] (one token) or row-major [T, C] (seq mode).
 *   - matrix weights are held on the device OUTPUT-MAJOR: element (k, n) of the
 *     reference's row-major [K=in, N=out] tensor (tools/convert_weight.py:44-46,
 *     kernels/cuda/matmul.cpp:105-121) lives at data[n*K + k].  frhip_pack_* produce
 *     that layout from the reference's.  A wavefront then streams whole rows of K
 *     contiguous elements and reduces them with cross-lane adds, and the prefill
 *     GEMM reads both operands K-contiguous.
 */
#ifndef FRHIP_H_
#define FRHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FRHIP_ABI_VERSION 1

enum {
  FRHIP_EINVAL = -1,  /* bad argument (null pointer, negative size, unknown enum) */
  FRHIP_ESHAPE = -2,  /* shape not supported by the kernel (alignment, maximum)  */
  FRHIP_ESTATE = -3,  /* call not valid now (e.g. graph capture not in progress)  */
  FRHIP_ENODEV = -4   /* no usable gfx950 device                                  */
};

enum { FRHIP_F32 = 0, FRHIP_F16 = 1, FRHIP_U8 = 2 };
enum { FRHIP_H2D = 0, FRHIP_D2H = 1, FRHIP_D2D = 2 };

typedef void *frhip_stream;
typedef void *frhip_event;
typedef void *frhip_graph;

/* A matrix weight as the kernels consume it.  For FRHIP_U8 the ChatRWKV-style
 * per-column (mx, rx: [N]) and per-row (my, ry: [K]) binary16 offsets and ranges
 * accompany the codes (parameters named at kernels/kernels.h:11-13); for FRHIP_F16
 * they are NULL. */
typedef struct frhip_weight {
  const void *data; /* [N][K] output-major, binary16 or uint8 */
  const void *mx, *rx; /* [N] binary16 */
  const void *my, *ry; /* [K] binary16 */
  int32_t K, N;
  int32_t dtype; /* FRHIP_F16 or FRHIP_U8 */
} frhip_weight;

/* ---- runtime: replaces the cudart calls of tensor.cpp:58-96 and the raw
 *      cudaMalloc/cudaFree under kernels/cuda/allocator.cpp:412-460 ------------- */
int frhip_abi_version(void);
const char *frhip_error_string(void);
int frhip_device_count(int *count);
int frhip_init(int device);                         /* select device, create handles; also lets this device's long-row
                                                       kernels use more than 64 KB of LDS (K beyond 32768 fp16 elements) */
int frhip_device_info(char *name, size_t name_len, int *compute_units, size_t *total_mem);
int frhip_malloc(void **ptr, size_t bytes);         /* hipMalloc; caching sits above, in the host allocator */
int frhip_free(void *ptr);
int frhip_host_malloc(void **ptr, size_t bytes);    /* pinned host memory for logits read-back */
int frhip_host_free(void *ptr);
int frhip_memcpy(void *dst, const void *src, size_t bytes, int kind);              /* blocking, as cudaMemcpy at tensor.cpp:65-73 */
int frhip_memcpy_async(void *dst, const void *src, size_t bytes, int kind, frhip_stream s);
int frhip_memset_async(void *dst, int byte, size_t bytes, frhip_stream s);
int frhip_stream_create(frhip_stream *s);
int frhip_stream_destroy(frhip_stream s);
int frhip_stream_sync(frhip_stream s);
int frhip_device_sync(void);
int frhip_event_create(frhip_event *e);
int frhip_event_destroy(frhip_event e);
int frhip_event_record(frhip_event e, frhip_stream s);
int frhip_event_sync(frhip_event e);
int frhip_event_elapsed_ms(frhip_event start, frhip_event stop, float *ms);
/* Capture everything launched on `s` between begin and end into a replayable graph
 * (the reference issues ~415 launches per token, kernels/default/model_forward.cpp:105-188). */
int frhip_graph_begin(frhip_stream s);
int frhip_graph_end(frhip_stream s, frhip_graph *g);
int frhip_graph_launch(frhip_graph g, frhip_stream s);
int frhip_graph_destroy(frhip_graph g);

/* ---- weight preparation ---------------------------------------------------- */
/* src: the reference's [K][N] row-major matrix on the device; dst: [N][K].
 * elem_bytes 1 (uint8 codes) or 2 (binary16). */
int frhip_pack_transpose(const void *src_kn, void *dst_nk, int K, int N, int elem_bytes, frhip_stream s);
/* Dequantise a packed uint8 weight into packed binary16, dst [N][K].  Evaluated in
 * IEEE binary32 with one final round-to-nearest-even to binary16:
 *   c = rx[n] / 255;  a = c * ry[k];  b = mx[n] + my[k];  w^ = h(fmaf(q, a, b)).
 * frhip_gemm multiplies by exactly this w^; the one-token operators (frhip_gemv, att, ffn,
 * head) evaluate the same formula in fp32 without the final rounding of w^. */
int frhip_dequant_u8(const frhip_weight *w, void *dst_nk_f16, frhip_stream s);
/* From this many rows on, the *_seq operators multiply uint8 weights by expanding them to binary16
 * first (into their workspace, once per call; below, and in frhip_gemm, which has no workspace,
 * the codes are dequantised on their way into the product).  A caller with memory to spare can
 * keep the frhip_dequant_u8 image of a weight and pass it as an FRHIP_F16 weight for such calls:
 * the products see the same w^ and the results are the same bits. */
#define FRHIP_SEQ_EXPAND_ROWS 4

/* ---- primitive operators (names of kernels/kernels.h) ------------------------ */
/* layernorm: kernels/cuda/layer_norm.cu:101-130.  dtype FRHIP_F16 or FRHIP_F32 for x, gamma, beta, y. */
int frhip_layernorm(const void *x, const void *gamma, const void *beta, void *y, int rows, int cols, int dtype, frhip_stream s);
/* groupnorm over fp32 rows: kernels/cuda/group_norm.cu:322-357. */
int frhip_groupnorm_f32(const float *x, int groups, const float *gamma, const float *beta, float *y, int rows, int cols, frhip_stream s);
/* matmul, vector x matrix: kernels/cuda/matmul.cpp:105-109.  x [K] binary16; y [N] in out_dtype (F16 or F32).
 * K a multiple of 16, at most 73728 for binary16 and 32768 for uint8 weights. */
int frhip_gemv(const void *x, const frhip_weight *w, void *y, int out_dtype, frhip_stream s);
/* cast_dtype: kernels/cuda/cast_dtype.cu:24-41. */
int frhip_cast(const void *src, int src_dtype, void *dst, int dst_dtype, size_t n, frhip_stream s);
/* fill_: kernels/cuda/fill.cu:17-27. */
int frhip_fill(void *x, int dtype, float value, size_t n, frhip_stream s);
/* scalar_div_: kernels/cuda/element_wise.cu:8-19 (binary16, divisor rounded to half first). */
int frhip_scalar_div_f16(void *x, float divisor, size_t n, frhip_stream s);
/* vgather of embedding rows: kernels/default/gather_ops.cpp:46-89.  table [V][C]; ids on the device. */
int frhip_gather_rows(const void *table, const int32_t *ids_dev, void *out, int n_ids, int row_bytes, frhip_stream s);

/* slice: kernels/cuda/slice.cu:38-136.  dst[i] = src[start + i * interval] per dimension, ndim 1..4;
 * the caller has resolved negative / whole-dimension ranges (slice.cu:54-66) into start, interval and
 * dst_shape.  Shapes travel as kernel arguments: no device allocation or blocking copy per call (the
 * reference makes four of each, slice.cu:79-111).  elem_bytes 1, 2 or 4. */
int frhip_slice(const void *src, void *dst, int ndim, const int *src_shape, const int *start, const int *interval,
                const int *dst_shape, int elem_bytes, frhip_stream s);
/* cat along one dimension: kernels/cuda/cat.cu:57-111.  a is [left][a_mid][right], b [left][b_mid][right]. */
int frhip_cat(const void *a, const void *b, void *out, size_t left, size_t a_mid, size_t b_mid, size_t right,
              int elem_bytes, frhip_stream s);
/* transpose of two dimensions: kernels/cuda/transpose.cu:36-103.  shape [ndim], ndim 1..4. */
int frhip_transpose(const void *src, void *dst, int ndim, const int *shape, int dim_a, int dim_b, int elem_bytes,
                    frhip_stream s);
/* silu: kernels/cuda/activations/silu.cu:38-57 in name and signature; the arithmetic is that of the
 * reference's fused path, x / (1 + half(exp(-x))) in half (kernels/cuda/att.cu:145-152) -- the
 * standalone reference kernel evaluates x / (1 - exp(x)) (silu.cu:19,28), which is not SiLU. */
int frhip_silu(const void *x, void *y, int dtype, size_t n, frhip_stream s);

/* Token feed for a replayed graph: reads ring[*counter % ring_len] (ring may be pinned host
 * memory, written by the host before the launch), advances *counter on the device, and copies
 * that row of `table` to `out`.  Ids outside [0, n_rows) are clamped.  Replaces the per-token
 * host-side row lookup `_embd_weights[id]` of kernels/default/model_forward.cpp:87, whose
 * pointer a captured graph could not change. */
int frhip_embed_ring(const void *table, int n_rows, int row_bytes, const int32_t *ring, int ring_len,
                     uint32_t *counter_dev, void *out, frhip_stream s);

/* Token feed of a greedy loop that the host does not take part in (the top_k = 1 case of
 * chat.cpp:56-92, where the host picks the token between two forward passes): the token is the
 * arg-max over `pairs`, the npairs {float value, int32 index} pairs frhip_argmax_blocks_f32 stored
 * for the previous step's logits (device or pinned host memory; greater value, then smaller
 * index; no finite maximum gives token 0).  It is stored to ids[*counter % ids_len] (device or
 * pinned host memory) for the host to read after a later synchronisation, *counter advances,
 * and that row of `table` is copied to `out`. */
int frhip_embed_argmax(const void *table, int n_rows, int row_bytes, const void *pairs, int npairs, int32_t *ids,
                       int ids_len, uint32_t *counter_dev, void *out, frhip_stream s);

/* ---- fused one-token operators ------------------------------------------------ */
/* Scratch the fused operators need: frhip_decode_workspace_bytes(C, F) bytes,
 * 256-byte aligned, owned by the caller, reusable across calls on one stream.
 * C (n_embd) is a multiple of 16 and at most 16384: up to 4096 an operator is two fused launches,
 * above that the same arithmetic runs as one launch per matrix (and the workspace holds the mixed
 * vectors).  F (n_ffn) is a multiple of 16, at most 73728 (binary16) / 32768 (uint8). */
size_t frhip_decode_workspace_bytes(int C, int F);

/* att (RWKV-4, one token): kernels/cuda/att.cu:182-217,337-359.
 * Reads x, sx [C] binary16; aa, bb, pp [C] fp32; writes x_out = x + out, xx_out =
 * LN(x) (the new shift state), aa_out, bb_out, pp_out.  aa_out/bb_out/pp_out may
 * alias aa/bb/pp and x_out may alias x; xx_out must not alias sx. */
int frhip_att_one_v4(int C, const void *x, const void *sx, const float *aa, const float *bb, const float *pp,
                     const void *ln_w, const void *ln_b, const void *k_mix, const void *v_mix, const void *r_mix,
                     const float *t_decay, const float *t_first,
                     const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw, const frhip_weight *ow,
                     void *x_out, void *xx_out, float *aa_out, float *bb_out, float *pp_out,
                     void *workspace, frhip_stream s);

/* ffn (one token): kernels/cuda/ffn.cu:62-110.  post_div2 != 0 additionally applies the
 * x /= 2 rescale of kernels/default/model_forward.cpp:173-175 to x_out. */
int frhip_ffn_one(int C, int F, const void *x, const void *sx, const void *ln_w, const void *ln_b,
                  const void *k_mix, const void *r_mix,
                  const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                  void *x_out, void *xx_out, int post_div2, void *workspace, frhip_stream s);

/* frhip_ffn_one without a workspace argument and without any allocation.  No counterpart in the
 * reference: it is for callers that cannot allocate device memory or hand over a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The
 * intermediate vectors (sigmoid(r) [C], relu(k)^2 [F]) live in a 112 KB device array built into the
 * library, one copy per GPU, held until the process ends.  Limits: C <= 4096, F <= 16384, else
 * FRHIP_ESHAPE.  All calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered.  Results are those of
 * frhip_ffn_one bit for bit. */
int frhip_ffn_one_static(int C, int F, const void *x, const void *sx, const void *ln_w, const void *ln_b,
                         const void *k_mix, const void *r_mix,
                         const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                         void *x_out, void *xx_out, int post_div2, frhip_stream s);

/* layernorm(ln_out) -> head matmul -> cast to fp32: kernels/default/model_forward.cpp:180-188. */
int frhip_head(int C, const void *x, const void *ln_w, const void *ln_b, const frhip_weight *head, float *logits, frhip_stream s);
/* The same with a second destination: every logit is also stored to mirror [N] (fp32), meant for pinned host
 * memory, so that the values cross the bus while the product runs instead of in a copy after it (the reference
 * copies after: tensor.cpp:65-68).  mirror may be null. */
int frhip_head_mirror(int C, const void *x, const void *ln_w, const void *ln_b, const frhip_weight *head, float *logits,
                      float *mirror, frhip_stream s);

/* att_one_v5_1 (RWKV-5.1/5.2, one token): kernels/cuda/att.cu:267-335,393-425.
 * s [H][S][S] fp32 ([head][key][value]); t_decay, t_first [H][S]; lx_w, lx_b [C] fp32.
 * s_out may alias s. */
int frhip_att_one_v5_1(int C, int H, const void *x, const void *sx, const float *s,
                       const void *ln_w, const void *ln_b, const float *lx_w, const float *lx_b,
                       const void *k_mix, const void *v_mix, const void *r_mix, const void *g_mix,
                       const float *t_decay, const float *t_first,
                       const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                       const frhip_weight *gw, const frhip_weight *ow,
                       void *x_out, void *xx_out, float *s_out, void *workspace, frhip_stream s_);

/* att_one_v5 (RWKV-5.0, one token): kernels/cuda/att.cu:219-265,362-391.  As
 * frhip_att_one_v5_1 without the gate; t_decay, t_first [H], one value per head
 * (att.cu:70,73 index them by i / (S*S)). */
int frhip_att_one_v5(int C, int H, const void *x, const void *sx, const float *s,
                     const void *ln_w, const void *ln_b, const float *lx_w, const float *lx_b,
                     const void *k_mix, const void *v_mix, const void *r_mix,
                     const float *t_decay, const float *t_first,
                     const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                     const frhip_weight *ow,
                     void *x_out, void *xx_out, float *s_out, void *workspace, frhip_stream s_);

/* ---- seq-mode (prompt) operators ---------------------------------------------- */
/* matmul, matrix x matrix: kernels/cuda/matmul.cpp:110-121.  x [T][K] binary16, y [T][N] in
 * out_dtype (F16 or F32); fp32 accumulation on the MFMA units.  K must be a multiple of 64. */
int frhip_gemm(const void *x, const frhip_weight *w, void *y, int T, int out_dtype, frhip_stream s);
/* matmul followed by the in-place activation the reference applies to its result, as one launch:
 * y [T][N] binary16 = act(half(x . w)).  act: FRHIP_ACT_SIGMOID (element_wise(InplaceSigmoid),
 * kernels/cuda/ffn_seq.cu:78-79, att.cu:154-159), FRHIP_ACT_RELU2 (InplaceReLUAndSquare,
 * ffn_seq.cu:80-81), FRHIP_ACT_SILU (InplaceSiLU, att_seq.cu:394-395, att.cu:145-152).  This is
 * the epilogue the seq operators below use for r, ffn key and the gate; results are theirs bit for bit. */
#define FRHIP_ACT_SIGMOID 2
#define FRHIP_ACT_RELU2 3
#define FRHIP_ACT_SILU 4
int frhip_gemm_act(const void *x, const frhip_weight *w, void *y, int T, int act, frhip_stream s);

/* Scratch for the seq-mode operators below: frhip_seq_workspace_bytes(T, C, F) bytes,
 * 256-byte aligned, owned by the caller. */
size_t frhip_seq_workspace_bytes(int T, int C, int F);

/* ffn_seq: kernels/cuda/ffn_seq.cu:65-109.  x, x_out [T][C]; sx [C]; xx_out [C] receives
 * LN(x)[T-1], the new shift state.  post_div2 as in frhip_ffn_one.  x_out may alias x. */
int frhip_ffn_seq(int T, int C, int F, const void *x, const void *sx, const void *ln_w, const void *ln_b,
                  const void *k_mix, const void *r_mix,
                  const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                  void *x_out, void *xx_out, int post_div2, void *workspace, frhip_stream s);

/* att_seq for RWKV-4.  The reference has no seq-mode att for version 4
 * (kernels/default/model_forward_seq.cpp:111-112 throws); its fallback
 * (model_forward_seq.cpp:34-46) defines the result as T one-token att steps
 * (kernels/cuda/att.cu:182-217), which is what this computes, with the products batched
 * over T and the WKV recurrence run as a chunked scan.  State arguments as frhip_att_one_v4. */
int frhip_att_seq_v4(int T, int C, const void *x, const void *sx, const float *aa, const float *bb, const float *pp,
                     const void *ln_w, const void *ln_b, const void *k_mix, const void *v_mix, const void *r_mix,
                     const float *t_decay, const float *t_first,
                     const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw, const frhip_weight *ow,
                     void *x_out, void *xx_out, float *aa_out, float *bb_out, float *pp_out,
                     void *workspace, frhip_stream s);

/* att_seq_v5_2: kernels/cuda/att_seq.cu:368-423,464-493.  State [H][S][S] indexed
 * [head][key][value] as in frhip_att_one_v5_1 (the reference transposes it around its scan
 * kernel, att_seq.cu:397,404; here the scan indexes it directly).  s_out may alias s. */
int frhip_att_seq_v5_2(int T, int C, int H, const void *x, const void *sx, const float *s,
                       const void *ln_w, const void *ln_b, const float *lx_w, const float *lx_b,
                       const void *k_mix, const void *v_mix, const void *r_mix, const void *g_mix,
                       const float *t_decay, const float *t_first,
                       const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                       const frhip_weight *gw, const frhip_weight *ow,
                       void *x_out, void *xx_out, float *s_out, void *workspace, frhip_stream s_);

/* att_seq_v5 (RWKV-5.0): kernels/cuda/att_seq.cu:158-256,425-462.  t_decay, t_first [H]. */
int frhip_att_seq_v5(int T, int C, int H, const void *x, const void *sx, const float *s,
                     const void *ln_w, const void *ln_b, const float *lx_w, const float *lx_b,
                     const void *k_mix, const void *v_mix, const void *r_mix,
                     const float *t_decay, const float *t_first,
                     const frhip_weight *kw, const frhip_weight *vw, const frhip_weight *rw,
                     const frhip_weight *ow,
                     void *x_out, void *xx_out, float *s_out, void *workspace, frhip_stream s_);

/* ---- bandwidth probes: DIAGNOSTICS, not operators (measurement aids of bench.py and of the
 *      hardware-counter calibration; no counterpart in the reference, nothing on the model path calls them) */
/* Plain device copy, 16 bytes per lane: the kernel of known traffic (bytes read + bytes
 * written) against which hardware counters are scaled. */
int frhip_copy_probe(void *dst, const void *src, size_t bytes, frhip_stream s);
/* Streams `bytes` of device memory once through the wavefronts (non-temporal 16-byte loads,
 * xor-folded so the loads are not dead) and writes one word per workgroup to `sink`
 * (at least 8192 bytes): the read-only ceiling the row-streaming kernels are compared with. */
int frhip_read_probe(const void *src, size_t bytes, void *sink, frhip_stream s);

/* Matrix-core rate probe: one workgroup of `waves_per_workgroup` (1..8) wavefronts per compute unit, each
 * issuing iters x 6 independent v_mfma_f32_32x32x16_f16 on register operands taken from `operands`
 * (4096 x 2 x 16 bytes of binary16: all zero, or random, which is what decides the clock the part
 * sustains).  sink: one float per thread; clocks: per wave {core-clock ticks, 100 MHz ticks} of the loop.
 * FLOP per launch = compute units x waves x iters x 6 x 32768. */
int frhip_mfma_probe(int waves_per_workgroup, int iters, const void *operands, void *sink, void *clocks, frhip_stream s);

/* greedy sampler step (Sampler::Sample with top_k = 1, chat.cpp:76-77): index of the
 * largest logit, first one on ties, written to *out_id on the device. */
int frhip_argmax_f32(const float *logits, int n, int32_t *out_id, frhip_stream s);
/* The same in two steps, for a loop that copies the logits to the host anyway: the first step on the
 * device over nblocks contiguous slices of x (16-byte aligned), writing nblocks pairs
 * {fp32 largest value of the slice, int32 index of its first occurrence} to `pairs` (device, 8 * nblocks
 * bytes; an empty slice reports -inf at index n); the second step, over the pairs (greater value,
 * then smaller index), is the caller's. */
int frhip_argmax_blocks_f32(const float *x, int n, void *pairs, int nblocks, frhip_stream s);
/* The same with the pairs stored twice: to `pairs` and, if not NULL, to `mirror` (e.g. `pairs` in device memory
 * for a next step that picks its token on the device, `mirror` in pinned host memory beside the logits the host
 * reads, chat.cpp:76-87). */
int frhip_argmax_blocks_f32_mirror(const float *x, int n, void *pairs, void *mirror, int nblocks, frhip_stream s);

#ifdef __cplusplus
}
#endif
#endif /* FRHIP_H_ */
