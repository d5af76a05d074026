/*
 * TEST INFRASTRUCTURE ONLY.  Scalar CPU restatement of the RWKV-7 inference hot path
 * (WKV7 recurrence, W8A16/W4A16 quantisation + GEMV, the fused element-wise ops, the
 * layer graph, the sampler's deterministic part).  It is the checker for the HIP
 * library and the timed CPU baseline; the shipped library never links or calls it.
 *
 * Every function cites the reference source it restates (paths relative to the
 * reference repository root).  fp16 tensors are passed as uint16_t bit patterns.
 *
 * Parity pins (what independent evidence each function is checked against, in tests/):
 *   - f16<->f32 conversion ........ numpy float16, exhaustive over all 65536 codes
 *   - wkv7 ........................ float64 brute force, closed-form special cases
 *   - wkv7, fp16 state ............ fp16 fma against exact rational arithmetic and numpy's float64 -> float16
 *                                   rounding; one-step closed forms (S = k v^T from an empty state, r = e_j reads
 *                                   column j of the new state), call-split invariance, the dither's range, known
 *                                   values and zero mean, agreement with the fp32-state recurrence to fp16 accuracy
 *   - LN / add+LN(+lerp) .......... float64 closed forms on the reference test's inputs
 *   - kk/a-gate, GroupNorm, v-res . float64 closed forms + special cases
 *   - gemv / lora ................. numpy matmul in float64
 *   - W8A16 / W4A16 format ........ PARITY UNPINNED at the reference boundary (the
 *                                   reference has no quantised path); pinned only by
 *                                   the format's own exhaustive code/round-trip tests
 *   - model graph ................. an independent float64 numpy restatement of the
 *                                   layer graph (tests/np_model.py)
 *   - sampler ..................... the reference sampler test's known answers
 */
#ifndef RWKV_ORACLE_H
#define RWKV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* number of worker threads used by the *_mt entry points and orc_model_forward (default 1) */
void orc_set_threads(int n);
int orc_get_threads(void);

/* ---- fp16 (round-to-nearest-even, as __float2half_rn) ------------------------------ */
uint16_t orc_f32_to_f16(float x);
float orc_f16_to_f32(uint16_t h);
void orc_f32_to_f16_array(const float* src, uint16_t* dst, int64_t n);
void orc_f16_to_f32_array(const uint16_t* src, float* dst, int64_t n);

/* checkpoint tensors: bf16 [rows,cols] -> fp16 (round to nearest even), optionally into [cols,rows];
 * embedding rows through LayerNorm(ln0) (cuda/rwkv7_v3a_ops.cu:70-116,153-185) */
void orc_bf16_to_f16(int rows, int cols, int transpose, const uint16_t* src, uint16_t* dst);
void orc_emb_ln0(int V, int C, const uint16_t* emb, const uint16_t* w, const uint16_t* b, float eps, uint16_t* out);

/* ---- WKV7 ---------------------------------------------------------------------------
 * state [B,H,64,64] f32 (row = value index i, column = key index j), in/out.
 * r,w,k,v,a,b,y [B,T,C].  w_mode 0: w is the raw decay logit, decay = exp(-e^-1/2 * sigmoid(w));
 * w_mode 1: w already holds the decay in (0,1). */
void orc_wkv7_f32(int B, int T, int C, int H, int w_mode, float* state,
                  const float* r, const float* w, const float* k, const float* v,
                  const float* a, const float* b, float* y);
void orc_wkv7_f16(int B, int T, int C, int H, int w_mode, float* state,
                  const uint16_t* r, const uint16_t* w, const uint16_t* k, const uint16_t* v,
                  const uint16_t* a, const uint16_t* b, uint16_t* y);

/* WKV7 with an fp16 state [B,H,64,64], every operation an fp16 fused multiply-add in the reference's order
 * (cuda/rwkv7_wkv_fp16_v2.cu:41-52,157-193).  w holds raw decay logits; w0 [C] (may be NULL) is added to them
 * unrounded; elapsed i32 [B] (tokens seen before this call) phases the decay dither and is not modified. */
void orc_wkv7_f16state(int B, int T, int C, int H, uint16_t* state, const uint16_t* r, const uint16_t* w,
                       const uint16_t* w0, const uint16_t* k, const uint16_t* v, const uint16_t* a,
                       const uint16_t* b, uint16_t* y, const int32_t* elapsed);
/* pieces of it, exported for the pin tests: double -> fp16 round-to-nearest-even, the fp16 fma, the dither
 * (:41-43) and the per-channel decay delta (:45-52) */
uint16_t orc_f64_to_f16(double x);
uint16_t orc_f16_fma(uint16_t a, uint16_t b, uint16_t c);
float orc_wkv16_rotator(int32_t x);
uint16_t orc_wkv16_w_delta(uint16_t w_raw, const uint16_t* w0, int c, int32_t phase);

/* ---- weight formats -----------------------------------------------------------------
 * W8A16: per-output-row symmetric int8, scale f16 [N].
 * W4A16: asymmetric 4-bit, groups of 128 along K, scale f16 [N,K/128], zero point u8 [N,K/128],
 *        codes packed two per byte (element k even -> low nibble of byte k/2). */
void orc_quantize_w8(int N, int K, const uint16_t* w, int8_t* q, uint16_t* scale);
void orc_dequant_w8(int N, int K, const int8_t* q, const uint16_t* scale, uint16_t* w);
void orc_quantize_w4(int N, int K, const uint16_t* w, uint8_t* q, uint16_t* scale, uint8_t* zp);
void orc_dequant_w4(int N, int K, const uint8_t* q, const uint16_t* scale, const uint8_t* zp, uint16_t* w);

/* y[M,N] = x[M,K] . W[N,K]^T, fp32 accumulate, f16 out. */
void orc_gemv_f16(int M, int N, int K, const uint16_t* x, const uint16_t* w, uint16_t* y);
void orc_gemv_w8(int M, int N, int K, const uint16_t* x, const int8_t* q, const uint16_t* scale, uint16_t* y);
void orc_gemv_w4(int M, int N, int K, const uint16_t* x, const uint8_t* q, const uint16_t* scale,
                 const uint8_t* zp, uint16_t* y);
/* same, fp32 result before the f16 rounding (for the lm_head) */
void orc_gemv_any_f32(int fmt, int M, int N, int K, const uint16_t* x, const void* w,
                      const uint16_t* scale, const uint8_t* zp, float* y);

/* ---- fused element-wise ops ---------------------------------------------------------- */
void orc_layer_norm(int rows, int C, const uint16_t* x, const uint16_t* w, const uint16_t* b,
                    uint16_t* y, float eps);
/* x_out = x + residual; y = LN(x + residual) (unrounded sum feeds the LN) */
void orc_add_layer_norm(int rows, int C, const uint16_t* x, const uint16_t* res, const uint16_t* w,
                        const uint16_t* b, uint16_t* x_out, uint16_t* y, float eps);
/* last token of each sequence only: y [B,C] */
void orc_add_last_layer_norm(int B, int T, int C, const uint16_t* x, const uint16_t* res,
                             const uint16_t* w, const uint16_t* b, uint16_t* y, float eps);
/* token-shift lerp: out_s = x + (prev - x) * mu_s, prev = shift[b] at t==0 else x[b,t-1];
 * then shift[b] = x[b,T-1].  n_mix mixes; mu [n_mix][C]; out [n_mix][B*T*C]. */
void orc_token_shift_mix(int B, int T, int C, int n_mix, const uint16_t* x, uint16_t* shift,
                         const uint16_t* const* mu, uint16_t* const* out);
/* T==1 fusions (rows = B): add + LN + lerp(s) + shift write */
void orc_add_layer_norm_cmix_mix(int rows, int C, const uint16_t* x, const uint16_t* res, uint16_t* shift,
                                 const uint16_t* w, const uint16_t* b, const uint16_t* mu_k,
                                 uint16_t* x_out, uint16_t* mixed, float eps);
void orc_add_layer_norm_tmix_mix6(int rows, int C, const uint16_t* x, const uint16_t* res, uint16_t* shift,
                                  const uint16_t* w, const uint16_t* b, const uint16_t* const* mu6,
                                  uint16_t* x_out, uint16_t* const* out6, float eps);
void orc_kk_a_gate(int rows, int C, int H, const uint16_t* k, const uint16_t* k_k, const uint16_t* a0,
                   const uint16_t* a12, const uint16_t* k_a, uint16_t* new_k, uint16_t* neg_kk, uint16_t* kka);
void orc_lnx_rkvres_xg(int rows, int C, int H, const uint16_t* y, const uint16_t* r, const uint16_t* k,
                       const uint16_t* v, const uint16_t* r_k, const uint16_t* lnw, const uint16_t* lnb,
                       const uint16_t* g, uint16_t* out);
/* v12 is fp32 (the unrounded LoRA output) */
void orc_vres_gate(int rows, int C, const uint16_t* v, const uint16_t* v_first, const uint16_t* v0,
                   const float* v12, uint16_t* out);
void orc_relu_square(int64_t n, const uint16_t* x, uint16_t* out);
void orc_add_vec(int rows, int C, const uint16_t* x, const uint16_t* vec, uint16_t* out);
/* LoRA: h = x . W1^T (W1 [R,C]) -> f16; out = act(h) . W2^T (W2 [C,R]) -> fp32.
 * act: 0 none, 1 tanh, 2 sigmoid. */
void orc_lora(int rows, int C, int R, int act, const uint16_t* x, const uint16_t* w1, const uint16_t* w2,
              float* out_f32);

/* ---- sampler (deterministic part) ---------------------------------------------------- */
/* logits' = (logits - penalties) / temperature; returns argmax (lowest index on ties);
 * then penalties = penalties*decay + (idx==tok ? (penalty==0 ? presence : frequency) : 0). */
int orc_sample_greedy_penalty(int V, const float* logits, float* penalties, float presence, float frequency,
                              float decay, float temperature);
/* probabilities after penalty/temperature/softmax and the top-k/top-p threshold filter:
 * writes probs[V] (zero outside the kept set, ties at the threshold scaled) and returns the
 * number of kept entries. */
int orc_sample_filter(int V, const float* logits, const float* penalties, float temperature, int top_k,
                      float top_p, float* probs);

/* ---- model graph ----------------------------------------------------------------------- */
enum {
  ORC_FMT_F16 = 0,
  ORC_FMT_W8 = 1,
  ORC_FMT_W4 = 2,
};
/* global tensors (layer = -1) */
enum {
  ORC_T_EMB_LN0 = 0, /* f16 [V,C], ln0 already applied */
  ORC_T_LN_OUT_W = 1,
  ORC_T_LN_OUT_B = 2,
  /* per layer vectors [C] */
  ORC_T_LN1_W = 10, ORC_T_LN1_B, ORC_T_LN2_W, ORC_T_LN2_B,
  ORC_T_X_R, ORC_T_X_W, ORC_T_X_K, ORC_T_X_V, ORC_T_X_A, ORC_T_X_G,
  ORC_T_W0, ORC_T_A0, ORC_T_V0, ORC_T_K_K, ORC_T_K_A, ORC_T_R_K, ORC_T_LNX_W, ORC_T_LNX_B, ORC_T_FFN_X_K,
  /* per layer LoRA, "out,in" layout: *1 is [R,C], *2 is [C,R] */
  ORC_T_W1 = 40, ORC_T_W2, ORC_T_A1, ORC_T_A2, ORC_T_G1, ORC_T_G2, ORC_T_V1, ORC_T_V2,
};
/* matrices [N_out,K_in] */
enum {
  ORC_M_ATT_R = 0, ORC_M_ATT_K, ORC_M_ATT_V, ORC_M_ATT_O, ORC_M_FFN_KEY, ORC_M_FFN_VALUE, ORC_M_HEAD,
};

typedef struct OrcModel OrcModel;
OrcModel* orc_model_create(int L, int C, int H, int F, int V, int Rw, int Ra, int Rg, int Rv);
void orc_model_destroy(OrcModel* m);
/* pointers are borrowed; the caller keeps the arrays alive */
int orc_model_set_tensor(OrcModel* m, int layer, int id, const uint16_t* data);
int orc_model_set_matrix(OrcModel* m, int layer, int id, int fmt, const void* data, const uint16_t* scale,
                         const uint8_t* zp);
/* tokens [B,T]; shift f16 [L,2,B,C]; wkv f32 [L,B,H,64,64]; elapsed i32 [B]; logits f32 [B,V]
 * (last token of each sequence).  trace, if not NULL, receives the residual stream after each
 * layer: f16 [L,B*T,C].  Returns 0, or a negative code on a bad argument. */
int orc_model_forward(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift, float* wkv,
                      int32_t* elapsed, float* logits, uint16_t* trace);
/* the same graph with the WKV state in fp16, wkv16 f16 [L,B,H,64,64] (src/rwkv7_fast_v4.cu:1266-1271) */
int orc_model_forward_f16state(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift,
                               uint16_t* wkv16, int32_t* elapsed, float* logits, uint16_t* trace);

#ifdef __cplusplus
}
#endif
#endif
