/*
 * rwkv_oracle.h -- CPU restatement of the RWKV forward pass of daquexian/faster-rwkv.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library may include, link or
 * call this file; it exists so that tests (and the bench's cpu_baseline leg) have
 * an independent statement of the arithmetic to compare the HIP path against.
 *
 * Two arithmetic modes are provided for every model-level function:
 *   ORC_F16  -- emulates the reference's CUDA fp16 path: every rounding to half
 *               that kernels/cuda/{att,ffn,att_seq,ffn_seq,layer_norm}.cu performs
 *               is performed here at the same point (round-to-nearest-even).
 *   ORC_F32  -- plain fp32, following the device-generic compositions in
 *               kernels/default/att.cpp and kernels/default/ffn.cpp.  This is the
 *               "kernels/cpu fp32 path" the reference never completed; it is the
 *               timed CPU baseline.
 *
 * Matrix weights are taken in the reference's storage order: row-major [in, out]
 * (tools/convert_weight.py:44-46, kernels/cuda/matmul.cpp:105-121).
 *
 * Parity status of each function (what pins it) is listed in oracle/README.md.
 * The uint8 dequantisation formula has no counterpart in the reference tree
 * (kernels/kernels.h:11-13 only names the mx/rx/my/ry parameters): PARITY UNPINNED
 * by the reference; it is pinned here by exhaustive evaluation against an
 * independent numpy statement of the same formula.  The same holds for orc_gemv_u8 (the
 * one-token product on unrounded fp32 weights): PARITY UNPINNED by the reference.
 */
#ifndef RWKV_ORACLE_H_
#define RWKV_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t orc_half; /* IEEE binary16 bit pattern */

enum { ORC_F32 = 0, ORC_F16 = 1 };

/* ---- binary16 scalar arithmetic (RTNE, subnormals kept) ------------------ */
orc_half orc_f2h(float f);
float orc_h2f(orc_half h);
orc_half orc_d2h(double d); /* correct single rounding double -> half */
orc_half orc_hadd(orc_half a, orc_half b);
orc_half orc_hsub(orc_half a, orc_half b);
orc_half orc_hmul(orc_half a, orc_half b);
orc_half orc_hdiv(orc_half a, orc_half b);
orc_half orc_hfma(orc_half a, orc_half b, orc_half c); /* single rounding */
void orc_f2h_n(const float *src, orc_half *dst, size_t n);
void orc_h2f_n(const orc_half *src, float *dst, size_t n);

/* ---- primitive ops ------------------------------------------------------- */
/* kernels/cuda/layer_norm.cu:33-80,101-130: fp32 statistics, eps 1e-5, biased
 * variance; in ORC_F16 the normalised value is rounded to half, multiplied by
 * gamma in half, then beta added in half. */
void orc_layernorm_f16(const orc_half *x, const orc_half *gamma, const orc_half *beta,
                       orc_half *y, int rows, int cols);
void orc_layernorm_f32(const float *x, const float *gamma, const float *beta, float *y,
                       int rows, int cols);
/* kernels/cuda/group_norm.cu:322-357: rows*groups instances of cols/groups. */
void orc_groupnorm_f32(const float *x, int groups, const float *gamma, const float *beta,
                       float *y, int rows, int cols);
/* kernels/cuda/att.cu:90-113, ffn.cu:15-32, att_seq.cu:21-45, ffn_seq.cu:16-34:
 * out = h(h(xx*m) + h(sx*h(1-m))); mix broadcast over rows (i % C). */
void orc_mix_f16(const orc_half *xx, const orc_half *sx, const orc_half *mix, orc_half *out,
                 int rows, int cols);
void orc_mix_f32(const float *xx, const float *sx, const float *mix, float *out, int rows,
                 int cols);
/* How orc_gemm_f16 accumulates.  The reference accumulates in fp32 in cuBLAS's own order
 * (kernels/cuda/matmul.cpp:38-42), which nothing pins; every such order lies within its own
 * rounding error of the exact sum.  ORC_ACC_EXACT (default) returns the centre of that family:
 * the exact sum rounded once to fp32.  ORC_ACC_F32_SEQUENTIAL is another member (fp32, ascending
 * k); running one model under both shows how far two valid evaluations of the reference's
 * arithmetic drift apart, i.e. the floor below which a logit tolerance cannot be met. */
enum { ORC_ACC_EXACT = 0, ORC_ACC_F32_SEQUENTIAL = 1 };
void orc_set_accumulation(int mode);
/* kernels/cuda/matmul.cpp:35-80: fp16 inputs, fp32 products and accumulation, one
 * rounding to the output type.  W is [K,N] row-major.  y_f32 or y_f16 may be NULL. */
void orc_gemm_f16(const orc_half *x, const orc_half *W, float *y_f32, orc_half *y_f16, int T,
                  int K, int N);
void orc_gemm_f32(const float *x, const float *W, float *y, int T, int K, int N);
/* kernels/cuda/att.cu:154-159 (double-precision exp, one rounding to half). */
void orc_sigmoid_f16(orc_half *x, size_t n);
/* kernels/cuda/ffn.cu:41-51. */
void orc_relu_square_f16(orc_half *x, size_t n);
/* kernels/cuda/att.cu:145-152. */
void orc_silu_f16(orc_half *x, size_t n);
/* kernels/cuda/att.cu:30-62.  r is in/out (half); state arrays updated in place. */
void orc_wkv4_one_f16(const float *t_first, const float *t_decay, const float *k,
                      const float *v, float *aa, float *bb, float *pp, orc_half *r, int n);

/* ---- uint8 weight-only quantisation (ChatRWKV-style mx/rx/my/ry) ---------- */
/* Dequantised weight, evaluated in IEEE binary32 with one final RTNE to binary16:
 *     c  = f32(rx[n]) / 255             (per output column n)
 *     a  = c * f32(ry[k])               (per element)
 *     b  = f32(mx[n]) + f32(my[k])
 *     w^ = h(fmaf(q, a, b))
 * (binary16 intermediates would put a relative error of 2^-12 on c, the same for a whole
 * column, which a product with same-signed activations does not average out.)
 * q is [K,N] row-major, mx,rx are [N] (per column), my,ry are [K] (per row). */
orc_half orc_dequant_u8_scalar(uint8_t q, orc_half mx, orc_half rx, orc_half my, orc_half ry);
void orc_dequant_u8(const uint8_t *q, const orc_half *mx, const orc_half *rx,
                    const orc_half *my, const orc_half *ry, orc_half *W, int K, int N);

/* The one-token product of the same scheme: every weight formed in fp32 by the formula above and
 * multiplied WITHOUT the rounding to half (products and sum exact in double, the sum rounded once
 * to fp32).  Follows the vector x matrix kernel of the ChatRWKV `rwkv` package (0.8.x,
 * rwkv/cuda/operators.cu, kernel_mm_one_fp16i8), which is not in the reference tree: PARITY
 * UNPINNED by the reference; pinned by float64 brute force of the real-valued formula and by
 * one-hot probes that must return fmaf(q, a, b) exactly. */
void orc_gemv_u8(const orc_half *x, const uint8_t *q, const orc_half *mx, const orc_half *rx,
                 const orc_half *my, const orc_half *ry, float *y, int K, int N);
/* After orc_register_u8(W, ...) every orc_gemm_f16 call with T == 1 on the binary16 matrix W
 * (the orc_dequant_u8 image of the codes) runs orc_gemv_u8 on the codes instead; calls with
 * T > 1 keep multiplying by W.  Keyed by pointer; the arrays must stay alive while registered. */
void orc_register_u8(const orc_half *W, const uint8_t *q, const orc_half *mx, const orc_half *rx,
                     const orc_half *my, const orc_half *ry);
void orc_unregister_u8(const orc_half *W);

/* ---- layer-level ops (one token) ----------------------------------------- */
/* kernels/cuda/att.cu:182-217,337-359.  x_out, xx_out [C]; aa,bb,pp updated in
 * place (the reference returns fresh tensors t1,t2,p that replace them). */
void orc_att_one_v4_f16(const orc_half *x, const orc_half *sx, float *aa, float *bb, float *pp,
                        const orc_half *ln_w, const orc_half *ln_b, const orc_half *k_mix,
                        const orc_half *v_mix, const orc_half *r_mix, const float *t_decay,
                        const float *t_first, const orc_half *kw, const orc_half *vw,
                        const orc_half *rw, const orc_half *ow, orc_half *x_out,
                        orc_half *xx_out, int C);
/* kernels/cuda/ffn.cu:62-110. */
void orc_ffn_one_f16(const orc_half *x, const orc_half *sx, const orc_half *ln_w,
                     const orc_half *ln_b, const orc_half *k_mix, const orc_half *r_mix,
                     const orc_half *kw, const orc_half *vw, const orc_half *rw, orc_half *x_out,
                     orc_half *xx_out, int C, int F);
/* kernels/cuda/att.cu:267-335,393-425 (serves v5.1 and v5.2).  s is [H,S,S] fp32
 * indexed [head][key][value], updated in place. u,w are [H,S]. */
void orc_att_one_v5_1_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                          const orc_half *ln_b, const float *lx_w, const float *lx_b,
                          const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                          const orc_half *g_mix, const float *t_decay, const float *t_first,
                          const orc_half *kw, const orc_half *vw, const orc_half *rw,
                          const orc_half *gw, const orc_half *ow, orc_half *x_out,
                          orc_half *xx_out, int C, int H);

/* kernels/cuda/att.cu:219-265,362-391 (RWKV-5.0: no gate; t_decay, t_first [H], one value
 * per head). */
void orc_att_one_v5_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                        const orc_half *ln_b, const float *lx_w, const float *lx_b,
                        const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                        const float *t_decay, const float *t_first, const orc_half *kw,
                        const orc_half *vw, const orc_half *rw, const orc_half *ow,
                        orc_half *x_out, orc_half *xx_out, int C, int H);

/* ---- layer-level ops (sequence of T tokens) ------------------------------ */
/* kernels/cuda/att_seq.cu:181-243: the RWKV-5.0 recurrence over T tokens in matrix form.
 * w, u [H]; s [H][S key][S value] updated in place; y [T][H*S]. */
void orc_wkv5_seq_matrix_f32(float *s, const float *r, const float *k, const float *v,
                             const float *w, const float *u, float *y, int T, int H, int S);
/* kernels/cuda/att_seq.cu:158-256,425-462. */
void orc_att_seq_v5_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                        const orc_half *ln_b, const float *lx_w, const float *lx_b,
                        const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                        const float *t_decay, const float *t_first, const orc_half *kw,
                        const orc_half *vw, const orc_half *rw, const orc_half *ow,
                        orc_half *x_out, orc_half *xx_last_out, int T, int C, int H);
/* kernels/cuda/ffn_seq.cu:65-109.  x [T,C]; sx [C] is the shift state; xx_last_out
 * receives LN(x)[T-1] (the new shift state). */
void orc_ffn_seq_f16(const orc_half *x, const orc_half *sx, const orc_half *ln_w,
                     const orc_half *ln_b, const orc_half *k_mix, const orc_half *r_mix,
                     const orc_half *kw, const orc_half *vw, const orc_half *rw, orc_half *x_out,
                     orc_half *xx_last_out, int T, int C, int F);
/* kernels/cuda/att_seq.cu:258-322 (scan) restated on the [head][key][value] state. */
void orc_wkv5_2_seq_f32(float *s, const float *r, const float *k, const float *v,
                        const float *w, const float *u, float *y, int T, int H, int S);
/* kernels/cuda/att_seq.cu:368-423,464-493. */
void orc_att_seq_v5_2_f16(const orc_half *x, const orc_half *sx, float *s, const orc_half *ln_w,
                          const orc_half *ln_b, const float *lx_w, const float *lx_b,
                          const orc_half *k_mix, const orc_half *v_mix, const orc_half *r_mix,
                          const orc_half *g_mix, const float *t_decay, const float *t_first,
                          const orc_half *kw, const orc_half *vw, const orc_half *rw,
                          const orc_half *gw, const orc_half *ow, orc_half *x_out,
                          orc_half *xx_last_out, int T, int C, int H);
/* RWKV-4 sequence attention.  The reference has none
 * (kernels/default/model_forward_seq.cpp:111-112 throws); its own fallback
 * (model_forward_seq.cpp:34-46) defines the result as T one-token steps, which is
 * what this does, with the matmuls batched over T. */
void orc_att_seq_v4_f16(const orc_half *x, const orc_half *sx, float *aa, float *bb, float *pp,
                        const orc_half *ln_w, const orc_half *ln_b, const orc_half *k_mix,
                        const orc_half *v_mix, const orc_half *r_mix, const float *t_decay,
                        const float *t_first, const orc_half *kw, const orc_half *vw,
                        const orc_half *rw, const orc_half *ow, orc_half *x_out,
                        orc_half *xx_last_out, int T, int C);

/* ---- whole model ---------------------------------------------------------- */
typedef struct {
  int version; /* 4, 50 (RWKV-5.0, ORC_F16 only) or 52 (RWKV-5.1/5.2) */
  int mode;    /* ORC_F32 or ORC_F16 */
  int n_layer, n_embd, n_att, n_ffn, n_head, vocab;
  /* Parameters in the reference's positional order
   * (kernels/default/init_model.cpp:91-126): per layer
   *   v4 : ln1.w ln1.b  tmk tmv tmr  time_decay time_first  Wk Wv Wr Wo
   *        ln2.w ln2.b  ffn.tmk ffn.tmr  ffn.Wk ffn.Wv ffn.Wr                (18)
   *   5.0: ln1.w ln1.b ln_x.w ln_x.b tmk tmv tmr time_decay time_first
   *        Wk Wv Wr Wo  ln2.w ln2.b ffn.tmk ffn.tmr ffn.Wk ffn.Wv ffn.Wr       (20)
   *   5.2: ln1.w ln1.b ln_x.w ln_x.b tmk tmv tmr tmg time_decay time_first
   *        Wk Wv Wr Wg Wo  ln2.w ln2.b ffn.tmk ffn.tmr ffn.Wk ffn.Wv ffn.Wr   (22)
   * then ln_out.w ln_out.b head.weight.
   * ORC_F16: time_decay, time_first, ln_x.* are float; everything else orc_half.
   * ORC_F32: everything float. */
  const void *const *params;
  const void *emb; /* [vocab, n_embd] */
} orc_model;

/* State: per layer, v4: sx_att[C] aa[C] bb[C] pp[C] sx_ffn[C]  (5 pointers)
 *                  5.2: sx_att[C] s[H,S,S] sx_ffn[C]           (3 pointers)
 * kernels/... model.cpp:145-177.  Shift states are orc_half (ORC_F16) or float. */
size_t orc_state_count(const orc_model *m);
void orc_state_reset(const orc_model *m, void *const *state);
size_t orc_state_elems(const orc_model *m, size_t idx);
int orc_state_is_act(const orc_model *m, size_t idx);

/* kernels/default/model_forward.cpp:22-193.  logits: [vocab] float. */
void orc_model_forward(const orc_model *m, void *const *state, int id, float *logits);
/* kernels/default/model_forward_seq.cpp:48-184 (last-token logits).  For v4 the
 * per-layer function is orc_att_seq_v4_f16. ORC_F32 models use the fallback loop. */
void orc_model_forward_seq(const orc_model *m, void *const *state, const int *ids, int T,
                           float *logits);
int orc_argmax(const float *x, int n);

#ifdef __cplusplus
}
#endif
#endif
