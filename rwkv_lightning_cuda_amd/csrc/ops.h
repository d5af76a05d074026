// Internal launcher interface shared by the op files and the model graph (not exported).
#pragma once

#include "common.h"

namespace rwkv {

// ---- linear.hip / gemm_mfma.hip ------------------------------------------------------------------
constexpr int kMaxProblems = 8;

struct LinearProblem {
  const void* w;
  const half_t* scale;
  const uint8_t* zp;
  const half_t* x;   // unused when the launch has a LayerNorm prologue
  void* y;
  int N;
  int fmt;           // RWKV_FMT_*
  const half_t* mu;  // with a LayerNorm prologue: this problem's token-shift lerp coefficients [K]
  // One-row launches without a LayerNorm prologue only: x = f16(x_f32 * x_gate) is formed while the block stages x
  // (the gate of the time-mix output, whose rank-out runs beside the heads' blocks instead of inside them).
  const float* x_f32 = nullptr;
  const half_t* x_gate = nullptr;
  // The few-row matrix-core launch only: a problem may be a slice of K columns of longer rows - values between the
  // starts of consecutive rows of W (ldw) and of x (ldx), 0 = K - and may leave its unscaled fp32 sums in y
  // (raw_f32: one of several slices' partial products, for a consumer that adds them up and scales).
  int ldw = 0;
  int ldx = 0;
  int raw_f32 = 0;
};

// LayerNorm + token-shift prologue of a small-M linear launch (decode steps): every block recomputes, for each
// of the M rows, s = x + res (or an embedding-table row), LN(s) and the lerp of this problem against the previous
// token's LN output, straight into its LDS copy of x - instead of a separate kernel writing six mixed copies of
// x that the linear kernel then reads back.  Arithmetic and reduction order are those of ln_fused_kernel.
// Block 0 also stores the residual sum and the LN output (the next shift row, written to the state by a later
// kernel so that no block can read a shift row that another block has already replaced).
struct LnPrologue {
  int mode = 0;  // 0 none, 1 residual add (x + res), 2 rows of `x` as a [V,K] table gathered by tokens, no residual
  const half_t* x = nullptr;
  const half_t* res = nullptr;
  const int64_t* tokens = nullptr;
  const half_t* w = nullptr;
  const half_t* b = nullptr;
  const half_t* shift = nullptr;  // [M,K], read only
  half_t* x_out = nullptr;        // [M,K] or NULL
  half_t* ln_out = nullptr;       // [M,K]
  float eps = 1e-5f;
};

// Extra duty of block 0 of a small-M linear launch: copy n fp16 values (the LN output kept by an earlier launch
// into its shift-state row).
struct RowCopy {
  const half_t* src = nullptr;
  half_t* dst = nullptr;
  int n = 0;
};

// Batched small-M linear through the weight-streaming kernels (the GEMV up to 8 rows; the few-row matrix-core
// launch from 5 to 16 rows where linear_rows_mfma_supported): up to kMaxProblems problems that share M and K (each
// with its own weight format, x and y) in one launch.
int linear_small_m(hipStream_t st, int M, int K, int n_problems, const LinearProblem* problems, int epilogue,
                   int out_f32, const LnPrologue* ln = nullptr, const RowCopy* copy = nullptr);
// Whether 5..16 rows of this format and shape run on the few-row matrix-core launch (weights in their plain order).
bool linear_rows_mfma_supported(int fmt, int N, int K);
// y = x W^T for rows of W longer than that launch takes (K a multiple of `slice`, a supported row length): one launch
// over K / slice column slices, whose fp32 partial sums [K / slice][M][N] go to `partial` for the consumer to add
// and scale (DeferredReduce).  M in 5..16.
int linear_rows_mfma_sliced(hipStream_t st, int fmt, int M, int N, int K, int slice, const half_t* x, const void* w,
                            float* partial, const RowCopy* copy = nullptr);
// Rows of a decode step that linear_small_m takes with the LayerNorm prologue at this row length (0: none): through
// the GEMV; and whether M rows of a format and shape go with it at all (the few-row matrix-core launch takes 5..8).
int linear_ln_prologue_max_rows(int K);
bool linear_ln_prologue_rows_ok(int fmt, int M, int N, int K);
// Any M: MFMA tiles for M >= 16 where supported, else row tiles through the GEMV kernel.
int linear_any_m(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* w, const half_t* scale,
                 const uint8_t* zp, int epilogue, int out_f32, void* y);
int linear_mfma(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* w, const half_t* scale,
                const uint8_t* zp, int epilogue, int out_f32, void* y);
bool linear_mfma_supported(int fmt, int M, int N, int K);

// ---- gemm_stream.hip: weights in the MFMA-native packed order ------------------------------------------------
bool linear_packed_supported(int fmt, int M, int N, int K);
// A packed linear call whose split-K partials are left for the consumer to sum (see LnArgs::res_partial).
// partial == NULL after the call: the shape needed no split and y holds the result.
struct DeferredReduce {
  const float* partial = nullptr;
  const half_t* scale = nullptr;
  int64_t plane = 0;
  int splits = 0;
};
int pack_weights_launch(hipStream_t st, int fmt, int N, int K, const void* w, void* packed);
// Workspace for one call: fp32 split-K partials (0 when the shape needs no split).
size_t linear_packed_workspace_bytes(int M, int N, int K);
// defer (single problem, fp16 output, no epilogue): the consumer sums the partials instead of a reduce launch.
int linear_packed(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* packed, const half_t* scale,
                  const uint8_t* zp, int epilogue, int out_f32, void* y, void* workspace, size_t workspace_bytes,
                  DeferredReduce* defer = nullptr, const RowCopy* copy = nullptr);
// Up to kMaxProblems products sharing M and K (own weights, format, x, y each) in one launch (+ one reduce launch).
struct PackedProblem {
  const void* packed;
  const half_t* scale;
  const uint8_t* zp;
  const half_t* x;
  void* y;
  int N;
  int fmt;
};
// Row counts and K at which a launch of int8 problems only gets a tile of its own (several wavefronts per SIMD):
// callers with int8 and fp16 problems for one launch do better with two launches there.
bool linear_packed_int8_tile(int M, int K);
size_t linear_packed_multi_workspace_bytes(int M, int K, int n_problems, const int* Ns);
int linear_packed_multi(hipStream_t st, int M, int K, int n_problems, const PackedProblem* problems, int epilogue,
                        int out_f32, void* workspace, size_t workspace_bytes, DeferredReduce* defer = nullptr,
                        const RowCopy* copy = nullptr);  // copy: rows moved by the launch's first block (n % 8 == 0)

// ---- fused_ops.hip ------------------------------------------------------------------------------
enum LnMode {
  kLn = 0,          // y = LN(x)
  kAddLn = 1,       // s = x + res; x_out = s; y = LN(s)
  kAddLastLn = 2,   // rows = B, reads row b*T + T-1; y only
  kAddLnMix = 3,    // kAddLn + n_mix lerps against shift, shift <- LN output (T == 1)
  kLnMix = 4,       // y = LN(x) without residual, then lerps + shift write (embedding row of layer 0)
  kAddLnMixSeq = 5, // kAddLn over rows [B,T] + n_mix lerps against the previous token's LN output (the shift row at
                    // t == 0); the LN output of each sequence's last token goes to shift_next, not to shift
};

struct LnArgs {
  const half_t* x;
  const half_t* res;
  const half_t* w;
  const half_t* b;
  half_t* x_out;
  half_t* y;
  half_t* shift;
  const half_t* mu[6];
  half_t* out[6];
  const int64_t* tokens;  // kLnMix: if not NULL, x is a [V,C] table indexed by tokens[row]
  half_t* shift_next;     // kAddLnMixSeq: [B,C], the next shift rows (the caller moves them into shift afterwards)
  int C;
  int T;
  int n_mix;
  float eps;
  // If res_partial is not NULL the residual is still the split-K partial tiles of a packed linear call:
  // res = f16(scale[c] * sum over splits of partial[s][row][c]), summed in split order (what the reduce
  // kernel of that call would have stored); `res` is then unused.
  const float* res_partial;
  const half_t* res_scale;  // NULL: no scale
  int64_t res_plane;        // elements between splits
  int res_splits;
};

int ln_launch(hipStream_t st, int mode, int rows, const LnArgs& a);

struct MixArgs {
  const half_t* x;
  half_t* shift;
  const half_t* mu[6];
  half_t* out[6];
  int B, T, C, n_mix;
};

int token_shift_mix_launch(hipStream_t st, const MixArgs& a);

struct KkArgs {
  const half_t* k;
  const half_t* k_k;
  const half_t* a0;
  const half_t* a12;
  const half_t* k_a;
  half_t* new_k;
  half_t* neg_kk;
  half_t* kka;
  // optional extras (all may be NULL): decay logits w12 (+ w0) and r, widened for the WKV kernel
  const half_t* w12;
  const half_t* w0;
  const half_t* r;
  float* k32;
  float* a32;
  float* b32;
  float* d32;
  float* r32;
  // optional (needs w12 and w0): f16(w12 + w0), the decay logit as the fp16-state recurrence takes it for calls of
  // more than 16 tokens (src/rwkv7_fast_v4.cu:1266-1271) - what add_vec_launch would write in a launch of its own
  half_t* w_sum16;
  int64_t rows_heads;
  int H;
};

int kk_a_gate_launch(hipStream_t st, const KkArgs& p);
int lnx_launch(hipStream_t st, int64_t rows_heads, int H, const half_t* y, const half_t* r, const half_t* k,
               const half_t* v, const half_t* r_k, const half_t* lnw, const half_t* lnb, const half_t* g, half_t* out);
int advance_launch(hipStream_t st, int n, int amount, int* x);
int add_vec_launch(hipStream_t st, int rows, int C, const half_t* x, const half_t* vec, half_t* out);  // out = f16(x + vec[c])
int embed_gather_launch(hipStream_t st, int rows, int C, const int64_t* tokens, const half_t* table, half_t* out);

// ---- lora.hip -----------------------------------------------------------------------------------
struct LoraOutProblem {
  const half_t* h;        // [M,R]
  const half_t* w2;       // [C,R]
  const half_t* w2p = nullptr;  // the same in the order of lora_pack_w2_launch (optional: coalesced weight reads)
  const half_t* bias;     // [C] or NULL
  const half_t* v;        // [M,C] (vres)
  const half_t* v_first;  // [M,C] (vres)
  half_t* out;            // [M,C]
  int R, act, vres;
};
struct LoraOutMultiArgs {
  LoraOutProblem p[4];
  int n, M, C;
};
// up to four rank-out products over the same rows in one launch
int lora_out_multi(hipStream_t st, const LoraOutMultiArgs& a);
// W2 [C,R] in the order the rank-out kernel's lanes read it: 32-channel bands x 16-wide rank steps x 64 lanes x 8
// values, lane (j, h) holding rank 16*step + 8*h .. + 8 of channel 32*band + j; zeros past C and R.
size_t lora_pack_w2_halfs(int C, int R);
int lora_pack_w2_launch(hipStream_t st, int C, int R, const half_t* w2, half_t* packed);

// ---- ffn_sparse.hip: one-token ffn.value product that skips the rows with a zero activation ---------------
bool ffn_sparse_supported(int fmt, int C, int F);  // fp16, int8 or int4 codes
size_t ffn_sparse_packed_bytes(int fmt, int C, int F);  // size of the transposed copy
// int4: codes [C,F/2] + scale / zp [C,F/128] -> codes [F,C/2], then scale and zp [F/128,C], in one allocation
int ffn_sparse_pack_w4_launch(hipStream_t st, int C, int F, const void* q, const half_t* scale, const uint8_t* zp, void* wt);
constexpr int kSparseMaxRows = 12;  // the reference's largest row count for this path (default_cmix_nofc_max_rows)
size_t ffn_sparse_workspace_bytes(int rows, int C, int F);
// [C,F] -> [F,C]; int8 codes are stored offset by 128
int ffn_sparse_pack_launch(hipStream_t st, int fmt, int C, int F, const void* w, void* wt);
// `in` [rows,F], `out` [rows,C].  activated != 0: `in` holds f16(relu(preact)^2) already; else the kernel applies it.
// `copy` (optional) rides on the second launch.  scale: per output channel for int8 codes, unused for fp16.
// one_walk: 2 .. kSparseUnionMaxRows tokens share one walk over the rows that are non-zero for any of them (each such
// row is read once); otherwise every token walks its own rows.
constexpr int kSparseUnionMaxRows = 4;
int ffn_sparse_launch(hipStream_t st, int fmt, int rows, int C, int F, int activated, const half_t* in, const void* wt,
                      const half_t* scale, void* workspace, size_t workspace_bytes, half_t* out, const RowCopy* copy,
                      bool one_walk);

// ---- sampler.hip --------------------------------------------------------------------------------
// out[b] = index of the largest logit of row b (the lowest one among equals); next / history (may be null) get the same id
int argmax_launch(hipStream_t st, int B, int V, const float* logits, int* out, int64_t* next = nullptr, int* history = nullptr);

// ---- wkv7.hip -----------------------------------------------------------------------------------
// T tokens of the recurrence from fp32 operands (decay applied); v, y fp16.  op_bs / io_bs: elements
// between batch rows of the operand / io tensors.
// The model's row-tiled time-mix pass in one launch: kk normalise / a-gate / decay while staging, the WKV recurrence,
// then per-head GroupNorm + (r.k.r_k) v bonus + gate on the way out.  All fp16 tensors [B,T,C] contiguous.
struct TmixSeqArgs {
  const half_t *r, *k, *a12, *w12, *g;
  const half_t *k_k, *a0, *k_a, *w0, *r_k, *lnx_w, *lnx_b;  // [C]
};
int tmix_seq_launch(hipStream_t st, int B, int T, int C, int H, float* state, const TmixSeqArgs& fa, const half_t* v,
                    half_t* y2);
// false: few heads in flight and more than one token - the stand-alone kernels are faster there (the recurrence
// then runs a head's row ranges on separate CUs, which the fused pass cannot: its GroupNorm needs whole heads)
bool tmix_seq_whole_heads(int B, int T, int H);
int wkv7_seq_f16_launch(hipStream_t st, int B, int T, int C, int H, float* state, const float* r, const float* d,
                        const float* k, const float* a, const float* b, int64_t op_bs, const half_t* v, half_t* y,
                        int64_t io_bs);

// ---- wkv7_f16state.hip: the recurrence with an fp16 state (w raw decay logits, w0 [C] or NULL added unrounded) ----
int wkv7_f16state_launch(hipStream_t st, int B, int T, int C, int H, half_t* state, const half_t* r, const half_t* w,
                         const half_t* w0, const half_t* k, const half_t* v, const half_t* a, const half_t* b, half_t* y,
                         const int* elapsed);

// One decode token per batch row with the fp16 state: kk normalise / a-gate, decay delta, the step, GroupNorm / bonus
// / gate in one launch (bitwise kk_a_gate + wkv7_f16state with T = 1 + lnx_rkvres_xg one after the other).
struct Tmix16RowsArgs {
  int64_t rows_heads;  // B * H
  int H;
  half_t* state;       // [B,H,64,64] fp16, updated in place
  const int* elapsed;  // [B]
  const half_t *r, *k, *v, *w12, *a12, *g;  // [B,C]; v after the residual gate, w12 / a12 / g the LoRA rank-outs
  const half_t *k_k, *a0, *k_a, *w0, *r_k, *lnx_w, *lnx_b;  // [C]
  half_t* y2;          // [B,C] input of the output projection
};
int tmix16_rows_launch(hipStream_t st, const Tmix16RowsArgs& p);

}  // namespace rwkv

namespace rwkv {

// ---- tmix_step.hip: the whole time-mix core of a decode step, one workgroup per head and 1, 2 or 4 batch rows ----
struct TmixStepArgs {
  int B, H, C, Rw, Ra, Rg, Rv;
  const half_t *hw, *ha, *hg, *hv;          // LoRA hidden vectors [B,R]; hv == NULL on layer 0
  const half_t *w2, *a2, *g2, *v2;          // LoRA rank-out matrices [C,R]
  const half_t *w0, *a0, *v0, *k_k, *k_a, *r_k, *lnx_w, *lnx_b;
  const half_t *r, *k, *v;                  // projections [B,C]
  const half_t* v_first;                    // [B,C], read when hv != NULL
  half_t* v_first_out;                      // [B,C], written when hv == NULL (layer 0), may be NULL
  float* state;                             // [B,H,64,64], updated in place (fp32-state mode)
  half_t* state16;                          // fp16-state mode (state == NULL): [B,H,64,64] in fp16 ...
  const int* elapsed;                       // ... and the tokens each row has seen, [B] (the decay's dither phase)
  half_t* y2;                               // [B,C] input of the output projection
  // Split mode (gate_out != NULL): the g rank-out - more than half of the launch's bytes - runs in B*H further
  // blocks that write the gate to gate_out [B,C]; the heads' blocks write the ungated output in fp32 to y2_pre
  // [B,C] instead of y2, and the consumer forms f16(y2_pre * gate) (the same product, rounded once).
  float* y2_pre;
  half_t* gate_out;
  const half_t* shift_src;                  // [B,C] LN output kept by the r/k/v launch's prologue, or NULL
  half_t* shift_dst;                        // [B,C] time-mix shift row of the state that receives it
  int rows_per_block;                       // batch rows of a head per block: 1, 2 or 4 (dividing B); 0 = chosen here
};
int tmix_step_launch(hipStream_t st, const TmixStepArgs& p);
// the choice that rows_per_block == 0 stands for (one_row_only: split mode or the fp16 state)
int tmix_step_rows_per_block(int B, int H, bool one_row_only);

}  // namespace rwkv
