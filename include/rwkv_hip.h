/*
 * C ABI of the MI355X (gfx950) RWKV-7 inference kernels.
 *
 * Plain pointers and sizes only: no HIP, CUDA or torch types.  Every `void*` tensor argument
 * is a device address unless the name ends in `_host`.  fp16 tensors are IEEE binary16.
 * `rwkv_stream_t` is an opaque stream handle (NULL = the default stream).
 *
 * Every function returns 0 on success or a negative RWKV_E_* code and never terminates the
 * process; rwkv_hip_last_error() returns the calling thread's last message.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference repository root).  The reference's kernel ABI is the C++-linkage launcher list in
 * cuda/rwkv7_fast_v4_kernels.cuh:8-211 plus src/utils/sampling.h:10-46.
 */
#ifndef RWKV_HIP_H
#define RWKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* rwkv_stream_t;

enum {
  RWKV_OK = 0,
  RWKV_E_INVALID = -1,     /* bad argument / shape the kernels do not support */
  RWKV_E_RUNTIME = -2,     /* HIP runtime error */
  RWKV_E_NOMEM = -3,       /* device or host allocation failed */
  RWKV_E_STATE = -4,       /* object used before it was fully set up */
};

enum { RWKV_FMT_F16 = 0, RWKV_FMT_W8 = 1, RWKV_FMT_W4 = 2 };
enum { RWKV_W_RAW_LOGIT = 0, RWKV_W_DECAY = 1 };
enum { RWKV_IO_F16 = 0, RWKV_IO_F32 = 1 };
enum { RWKV_ACT_NONE = 0, RWKV_ACT_TANH = 1, RWKV_ACT_SIGMOID = 2 };
enum { RWKV_EPI_NONE = 0, RWKV_EPI_RELU_SQUARE = 1 };

const char* rwkv_hip_last_error(void);

/* ---- runtime plumbing.  Replaces the cudaMalloc/cudaMemcpy/cudaMemset/cudaStream* calls
 * inside DeviceBuffer<T> (include/rwkv7_fast_v4_common.hpp:64-110), run_backend_forward
 * (src/rwkv7_fast_v4.cu:1087-1096,1343-1344) and StateCacheManager
 * (src/rwkv_state_cache.cpp:132-223). ---- */
int rwkv_hip_device_count(int* count);
int rwkv_hip_device_name(char* buf, size_t buf_len);
int rwkv_hip_malloc(void** ptr, size_t bytes);
int rwkv_hip_free(void* ptr);
/* Blocks that come back: rwkv_hip_free_recycled keeps the block (after waiting for the device, as hipFree does) and
 * the next rwkv_hip_malloc_recycled of the same byte size on the same device returns it - last in, first out, not
 * cleared.  The generation state and logits of consecutive requests of one shape then sit at the same addresses,
 * which is what a session's captured decode graphs are keyed by.  At most 24 GiB are held (oldest freed first);
 * an allocation that fails for lack of memory frees them all and tries again; rwkv_hip_mem_info counts them as
 * free; rwkv_hip_recycle_trim frees them.  No counterpart in the reference (cudaMalloc / cudaFree per
 * DeviceBuffer, include/rwkv7_fast_v4_common.hpp:64-110). */
int rwkv_hip_malloc_recycled(void** ptr, size_t bytes);
int rwkv_hip_free_recycled(void* ptr, size_t bytes);
int rwkv_hip_recycle_trim(void);
int rwkv_hip_host_alloc(void** ptr_host, size_t bytes); /* pinned */
int rwkv_hip_host_free(void* ptr_host);
int rwkv_hip_memcpy_h2d(void* dst, const void* src_host, size_t bytes);
int rwkv_hip_memcpy_d2h(void* dst_host, const void* src, size_t bytes);
int rwkv_hip_memcpy_d2d(void* dst, const void* src, size_t bytes);
int rwkv_hip_memcpy_h2d_async(rwkv_stream_t s, void* dst, const void* src_host, size_t bytes);
int rwkv_hip_memcpy_d2h_async(rwkv_stream_t s, void* dst_host, const void* src, size_t bytes);
int rwkv_hip_memcpy_d2d_async(rwkv_stream_t s, void* dst, const void* src, size_t bytes);
int rwkv_hip_memset(void* ptr, int value, size_t bytes);
int rwkv_hip_mem_info(size_t* free_bytes, size_t* total_bytes);
int rwkv_hip_stream_create(rwkv_stream_t* s);
int rwkv_hip_stream_destroy(rwkv_stream_t s);
int rwkv_hip_stream_sync(rwkv_stream_t s);
int rwkv_hip_device_sync(void);
/* event timing on a stream: ms between two recorded points, for benchmarks */
int rwkv_hip_event_create(void** ev);
int rwkv_hip_event_destroy(void* ev);
int rwkv_hip_event_record(void* ev, rwkv_stream_t s);
int rwkv_hip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms);
/* ordering between streams and with the host, for pipelines that copy on one stream and compute on another (the
 * checkpoint loader; the reference pairs copy and compute streams the same way, src/rwkv7_fast_v4.cu:110-181):
 * the host waits for a recorded event; work enqueued on `s` after the call starts only once the event has happened */
int rwkv_hip_event_sync(void* ev);
int rwkv_hip_stream_wait_event(rwkv_stream_t s, void* ev);

/* Measurement aid (no counterpart in the reference): the cost of a launch that has to wait for its predecessor.
 * Runs a chain of `links` launches of a kernel that does next to nothing (every block reads a counter, one thread
 * writes it back incremented) with `blocks` x `threads` each, on a stream of its own, `reps` times after one warm
 * run - as direct launches or as one captured graph per run - and returns the microseconds per link.  A decode step
 * at batch 1 is such a chain (8 launches per layer); this is the part of its time that no kernel can remove. */
int rwkv_hip_measure_launch_chain(int links, int blocks, int threads, int use_graph, int reps, float* us_per_link);

/* ---- WKV7 time-mix recurrence.  Replaces rwkv7_wkv_fp32io16_launch
 * (cuda/rwkv7_fast_v4_kernels.cuh:49-52, cuda/rwkv7_wkv_fp32_v2.cu:237-294).
 * state f32 [B,H,64,64] in/out; r,w,k,v,a,b,y [B,T,C], C == H*64.
 * w_mode RWKV_W_RAW_LOGIT: decay = exp(-e^-1/2 * sigmoid(w)) (the reference's only mode);
 * RWKV_W_DECAY: w is the decay itself.  io RWKV_IO_F16 / RWKV_IO_F32 selects the element type of
 * r..y (the reference builds one or the other with _IO_FP16_, rwkv7_wkv_fp32_v2.cu:16-24).
 * Running T1+T2 tokens in one call or in two consecutive calls gives bitwise the same result. */
int rwkv_hip_wkv7(rwkv_stream_t s, int B, int T, int C, int H, int w_mode, int io, void* state,
                  const void* r, const void* w, const void* k, const void* v, const void* a, const void* b,
                  void* y);

/* The recurrence with the state kept in fp16 (the reference server's default; ModelBackend's use_wkv32 == false).
 * Replaces rwkv7_wkv_fp16_seq_launch / rwkv7_wkv_fp16_seq_w0_launch and the one-token launchers
 * (cuda/rwkv7_fast_v4_kernels.cuh:34-47, cuda/rwkv7_wkv_fp16_v2.cu:681-830).  state f16 [B,H,64,64] in/out;
 * r,w,k,v,a,b,y f16 [B,T,C]; w holds raw decay logits, w0 f16 [C] (may be NULL) is added to them unrounded;
 * elapsed i32 [B] = tokens each row has seen before this call (read only: it phases the dither that the
 * reference adds to the decay before rounding it to fp16, cuda/rwkv7_wkv_fp16_v2.cu:41-52).  Every operation is an
 * fp16 fused multiply-add in the reference's order.  T1+T2 tokens in one call or in two (elapsed advanced by T1
 * in between) give bitwise the same result, and so does any batch size (the kernel gives a state row to four, two
 * or one lanes by the number of heads in the call; the sums keep their order).  T * C must stay below 2^31. */
int rwkv_hip_wkv7_f16state(rwkv_stream_t s, int B, int T, int C, int H, void* state, const void* r, const void* w,
                           const void* w0, const void* k, const void* v, const void* a, const void* b, void* y,
                           const void* elapsed);

/* ---- weight formats (no counterpart in the reference, whose weights are fp16 only).
 * W8: int8 [N,K] + f16 scale [N].  W4: packed u8 [N,K/2] (element k even -> low nibble of byte
 * k/2) + f16 scale [N,K/128] + u8 zero point [N,K/128]; K % 128 == 0. ---- */
int rwkv_hip_quantize_w8(rwkv_stream_t s, int N, int K, const void* w_f16, void* q, void* scale);
int rwkv_hip_dequant_w8(rwkv_stream_t s, int N, int K, const void* q, const void* scale, void* w_f16);
int rwkv_hip_quantize_w4(rwkv_stream_t s, int N, int K, const void* w_f16, void* q, void* scale, void* zp);
int rwkv_hip_dequant_w4(rwkv_stream_t s, int N, int K, const void* q, const void* scale, const void* zp,
                        void* w_f16);

/* ---- checkpoint tensors: bf16 in the file, fp16 on the device.  Replace rwkv7_v4_bf16_to_f16_launch,
 * rwkv7_v4_bf16_to_f16_transpose_launch and rwkv7_v4_emb_ln0_bf16_to_f16_launch
 * (cuda/rwkv7_fast_v4_kernels.cuh:8-29): widening to fp32 is exact, the fp16 result is rounded to nearest even.
 * transpose: src [rows,cols] -> dst [cols,rows].  emb_ln0: out[v] = f16(LayerNorm(emb[v]) * weight + bias) with
 * two-pass fp32 statistics, emb [V,C], weight / bias [C] all bf16. ---- */
int rwkv_hip_bf16_to_f16(rwkv_stream_t s, int64_t n, const void* src_bf16, void* dst_f16);
int rwkv_hip_bf16_to_f16_transpose(rwkv_stream_t s, int rows, int cols, const void* src_bf16, void* dst_f16);
int rwkv_hip_emb_ln0_bf16_to_f16(rwkv_stream_t s, int V, int C, const void* emb_bf16, const void* weight_bf16,
                                 const void* bias_bf16, float eps, void* out_f16);

/* Synthetic fp16 weights ~ mean + std*N(0,1) from a counter-based hash of (seed, index): random-init
 * models for benchmarks without a checkpoint (no counterpart in the reference, which loads .pth files). */
int rwkv_hip_fill_normal_f16(rwkv_stream_t s, int64_t n, uint64_t seed, float mean, float stdv, void* out);

/* ---- linear layers, y[M,N] = x[M,K] . W[N,K]^T, fp32 accumulate.
 * Replaces rwkv7_v3a_linear_orig_rows_exact_f16_launch / _orig_rows_f16_launch / _f16_orig_launch /
 * _f16_orig_lt_cfg_launch (cuda/rwkv7_fast_v4_kernels.cuh:155-177) and the dispatch in
 * linear_orig_layout_launch (src/rwkv7_fast_v4.cu:709-959).  Any M: up to 4 rows stream the weights
 * once through a GEMV kernel that keeps whole weight rows in flight; 5 to 16 rows of int8 / fp16
 * weights with K a multiple of 1024 up to 4096 stream them the same way with the products on the
 * matrix core; otherwise up to 8 rows per pass of a GEMV with K tiles, and from 16 rows MFMA tiles.
 * out_f32 == 0: y is f16 [M,N].  out_f32 == 1: y is f32 [M,N] holding the f16-rounded value
 * (the lm_head path, src/rwkv7_fast_v4.cu:1325-1341 + rwkv7_v4_f16_to_f32_launch).
 * epilogue RWKV_EPI_RELU_SQUARE applies relu(.)^2 to the f16-rounded result and rounds again
 * (rwkv7_relu_square_launch, cuda/rwkv7_fast_v4_kernels.cuh:83). */
int rwkv_hip_linear(rwkv_stream_t s, int fmt, int M, int N, int K, const void* x, const void* w,
                    const void* scale, const void* zp, int epilogue, int out_f32, void* y);

/* The same product over weights in the MFMA-native packed order: the path for M >= 16 (prefill chunks
 * and batched decode; the reference sends these to cuBLAS / cuBLASLt,
 * cuda/rwkv7_v3a_ops.cu:2235-2368, with per-shape algorithm ids at src/rwkv7_fast_v4.cu:753-958).
 * rwkv_hip_pack_weights permutes the 16-byte pieces of row-major codes w [N,K] (fp16, int8 or int4 as
 * for rwkv_hip_linear) into `packed` (same byte count, must not alias w); scale and zp keep their
 * row-major layout.  Requires N % 32 == 0 and K % 256 == 0.  The workspace holds fp32 split-K
 * partial sums; rwkv_hip_linear_packed_workspace gives the size for a shape (0 when the shape is not
 * split; workspace may then be NULL).  Calls sharing one workspace must not overlap.  Results do not
 * depend on scheduling (partials are summed in a fixed order). */
int rwkv_hip_pack_weights(rwkv_stream_t s, int fmt, int N, int K, const void* w, void* packed);
int rwkv_hip_linear_packed_workspace(int M, int N, int K, size_t* bytes);
int rwkv_hip_linear_packed(rwkv_stream_t s, int fmt, int M, int N, int K, const void* x, const void* packed,
                           const void* scale, const void* zp, int epilogue, int out_f32, void* y,
                           void* workspace, size_t workspace_bytes);

/* ---- ffn.value of a few tokens, reading per token only the rows with a non-zero activation.  Replaces
 * rwkv7_cmix_sparse_down_relu_one_launch and rwkv7_cmix_sparse_down_relu_rows_launch
 * (cuda/rwkv7_fast_v4_kernels.cuh:90-100, cuda/rwkv7_fast_ops_fp16.cu:966-992,618-737), per token:
 *   vec[f] = f16(relu(preact[f])^2);  out[c] = f16(sum over f with vec[f] != 0 of vec[f] * W[c][f])
 * for fmt = RWKV_FMT_F16 (the reference's case), or with int8 codes (RWKV_FMT_W8)
 *   out[c] = f16(scale[c] * sum over f with vec[f] != 0 of vec[f] * q[c][f]).
 * preact [rows,F], out [rows,C], rows 1..12.  The reference accumulates in half2 with atomicAdd; this one
 * accumulates exact products in fp32 in a fixed order, so it equals the dense product up to fp32 summation order
 * and repeats bitwise.
 * cmix_sparse_pack turns the [C,F] matrix (fp16 values, or the codes of rwkv_hip_quantize_w8) into the [F,C]
 * copy `wt` (same size) that the product reads - the layout the reference keeps ffn.value in
 * (include/rwkv7_fast_v4_common.hpp:313-321); `scale` is the per-output-channel tensor of the codes (unused
 * for fp16).  C % 16 == 0, F % 256 == 0.  workspace: fp32 partial rows, size from cmix_sparse_workspace.
 * int4 codes (RWKV_FMT_W4, groups of 128 along F; no counterpart in the reference):
 *   out[c] = f16(sum over groups g of scale[c][g] * sum over f in g with vec[f] != 0 of vec[f] * (q[c][f] - zp[c][g]));
 * cmix_sparse_pack_w4 writes the codes [F,C/2], then the scales and zero points transposed to [F/128,C], into one
 * allocation `wt` of cmix_sparse_packed_bytes; the product then ignores its `scale` argument. */
int rwkv_hip_cmix_sparse_pack(rwkv_stream_t s, int fmt, int C, int F, const void* w, void* wt);
int rwkv_hip_cmix_sparse_pack_w4(rwkv_stream_t s, int C, int F, const void* q, const void* scale, const void* zp,
                                 void* wt);
int rwkv_hip_cmix_sparse_packed_bytes(int fmt, int C, int F, size_t* bytes);
int rwkv_hip_cmix_sparse_workspace(int rows, int C, int F, size_t* bytes);
int rwkv_hip_cmix_sparse_down_relu_rows(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                        const void* wt, const void* scale, void* workspace, size_t workspace_bytes,
                                        void* out);
int rwkv_hip_cmix_sparse_down_relu_one(rwkv_stream_t s, int fmt, int C, int F, const void* preact, const void* wt,
                                       const void* scale, void* workspace, size_t workspace_bytes, void* out);
/* The same product for 2..4 tokens that share one walk over the matrix: every row that is non-zero for any of the
 * tokens is read once (a token for which it is zero takes it with an exact zero coefficient), where the _rows call
 * reads it once per token that needs it - the form the reference's rows kernel has
 * (cmix_sparse_spmv_relu_rows_kernel, cuda/rwkv7_fast_ops_fp16.cu:681-737: one block walks a row tile for all
 * rows of the batch).  Same arguments and workspace as _rows.  Per token the rows add up in increasing order, but
 * pair up differently than in the token's own walk, so the result equals _rows up to the last bits of the fp32
 * sums; it repeats bitwise from call to call. */
int rwkv_hip_cmix_sparse_down_relu_rows_shared(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                               const void* wt, const void* scale, void* workspace,
                                               size_t workspace_bytes, void* out);
/* The same product as rwkv_hip_cmix_sparse_down_relu_rows (same kernels, bitwise the same result) for callers
 * that cannot allocate or bring a workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference.  The fp32 partial rows live in a 16 MiB array that is part
 * of the library's device image (one copy per GPU, held until the process ends); the call allocates and frees
 * nothing.  rows * (F / 256) * C * 4 bytes must fit in it (7.2B shape: all 12 rows), else RWKV_E_INVALID.  Every
 * call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls
 * on one stream are ordered.  Nothing in the array needs clearing between calls (every partial row that is read
 * has been written by the same call).  The first call on a device looks up the array's device address
 * (hipGetSymbolAddress), so make it outside a stream capture. */
int rwkv_hip_cmix_sparse_down_relu_rows_static(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                               const void* wt, const void* scale, void* out);

/* ---- LoRA pairs.  Replaces rwkv7_v3a_linear_wag(v)_rank_in_f16_launch,
 * rwkv7_v3a_linear_wag(v)_rank_out_f16_launch, rwkv7_v3a_linear_t_f16_launch,
 * rwkv7_v3a_linear_t_act_f16_launch, rwkv7_v3a_linear_t_vres_f16_launch
 * (cuda/rwkv7_fast_v4_kernels.cuh:147-211).
 * lora_in:  h[M,R] = f16(x[M,C] . W1[R,C]^T).
 * lora_out: o[M,C] = act(h[M,R]) . W2[C,R]^T in fp32; then
 *   vres == 0: out = f16(o + bias[c])              (bias may be NULL: w0 folded for the decay logit)
 *   vres == 1: out = f16(v + (v_first - v) * sigmoid(bias[c] + o))   (the v-residual gate). */
int rwkv_hip_lora_in(rwkv_stream_t s, int M, int C, int R, const void* x, const void* w1, void* h);
int rwkv_hip_lora_out(rwkv_stream_t s, int M, int C, int R, int act, const void* h, const void* w2,
                      const void* bias, int vres, const void* v, const void* v_first, void* out);

/* ---- fused element-wise ops ---- */
/* rwkv7_v3a_layer_norm_f16_launch (cuda/rwkv7_fast_v4_kernels.cuh:118-120) */
int rwkv_hip_layer_norm(rwkv_stream_t s, int rows, int C, const void* x, const void* w, const void* b,
                        void* y, float eps);
/* rwkv7_v3a_add_layer_norm_f16_launch (:122-125) */
int rwkv_hip_add_layer_norm(rwkv_stream_t s, int rows, int C, const void* x, const void* res, const void* w,
                            const void* b, void* x_out, void* y, float eps);
/* rwkv7_v3a_add_last_layer_norm_f16_launch (:127-130): y [B,C] from the last token of each row */
int rwkv_hip_add_last_layer_norm(rwkv_stream_t s, int B, int T, int C, const void* x, const void* res,
                                 const void* w, const void* b, void* y, float eps);
/* rwkv7_tmix_mix6_launch (:54-60) and rwkv7_cmix_mix_launch (:79-81), including the shift-state
 * update.  n_mix in {1,6}; mu and out are host arrays of n_mix device pointers. */
int rwkv_hip_token_shift_mix(rwkv_stream_t s, int B, int T, int C, int n_mix, const void* x, void* shift,
                             const void* const* mu_host, void* const* out_host);
/* rwkv7_v3a_add_layer_norm_cmix_mix_f16_launch (:132-136); rows = B, T == 1 */
int rwkv_hip_add_layer_norm_cmix_mix(rwkv_stream_t s, int rows, int C, const void* x, const void* res,
                                     void* shift, const void* w, const void* b, const void* mu_k,
                                     void* x_out, void* mixed, float eps);
/* rwkv7_v3a_add_layer_norm_tmix_mix6_f16_launch (:138-145); rows = B, T == 1 */
int rwkv_hip_add_layer_norm_tmix_mix6(rwkv_stream_t s, int rows, int C, const void* x, const void* res,
                                      void* shift, const void* w, const void* b, const void* const* mu6_host,
                                      void* x_out, void* const* out6_host, float eps);
/* rwkv7_tmix_kk_a_gate_launch (:62-66) */
int rwkv_hip_kk_a_gate(rwkv_stream_t s, int rows, int C, int H, const void* k, const void* k_k, const void* a0,
                       const void* a12, const void* k_a, void* new_k, void* neg_kk, void* kka);
/* rwkv7_tmix_lnx_rkvres_xg_launch (:68-72) */
int rwkv_hip_lnx_rkvres_xg(rwkv_stream_t s, int rows, int C, int H, const void* y, const void* r, const void* k,
                           const void* v, const void* r_k, const void* lnw, const void* lnb, const void* g,
                           void* out);
/* rwkv7_relu_square_launch (:83), rwkv7_add_vec_launch (:87-88), rwkv7_v4_f16_to_f32_launch (:31-32),
 * rwkv7_v3a_advance_i32_launch (:116) */
int rwkv_hip_relu_square(rwkv_stream_t s, int64_t n, const void* x, void* out);
int rwkv_hip_add_vec(rwkv_stream_t s, int rows, int C, const void* x, const void* vec, void* out);
int rwkv_hip_f16_to_f32(rwkv_stream_t s, int64_t n, const void* src, void* dst);
int rwkv_hip_advance_i32(rwkv_stream_t s, int n, int amount, void* x);

/* ---- sampler.  Replaces rwkv_sampling::setup_rand_raw / batch_sampling_repetition_temperature_topk_topp_raw
 * / batch_sampling_temperature_topk_topp_raw (src/utils/sampling.h:14-46).
 * logits f32 [B,V]; penalties f32 [B,V] in/out (NULL = no penalty, as the no-penalty reference entry);
 * probs f32 [B,V] scratch; out i32 [B].  The random stream is a counter-based Philox4x32-10 keyed by
 * (seed, row, step): same arguments give the same tokens.  V % 4 == 0, V <= 1048576,
 * temperature in [0.001, 1000], as the reference checks (src/utils/sampling.cu:492-512). */
int rwkv_hip_sample(rwkv_stream_t s, int B, int V, const void* logits, void* penalties, void* probs, void* out,
                    double presence, double frequency, double decay, double temperature, int top_k,
                    double top_p, uint64_t seed, uint64_t step);
/* lm_head -> argmax without the sampler: out i32 [B] = lowest index of the row maximum */
int rwkv_hip_argmax(rwkv_stream_t s, int B, int V, const void* logits, void* out);

/* ---- model graph.  Replaces CudaWeights + run_backend_forward (src/rwkv7_fast_v4.cu:1046-1345) and
 * ModelBackend::{create_state,forward_prefill,forward_decode} (:1373-1419) below IModelBackend. ---- */
/* global tensors use layer = -1 */
enum {
  RWKV_T_EMB_LN0 = 0, /* f16 [V,C]: embedding with ln0 applied (build_cpu_emb_ln0_f16, src/rwkv7_fast_v4.cu:450-572) */
  RWKV_T_LN_OUT_W = 1,
  RWKV_T_LN_OUT_B = 2,
  /* per-layer f16 vectors [C] (LayerWeights, include/rwkv7_fast_v4_common.hpp:146-190) */
  RWKV_T_LN1_W = 10, RWKV_T_LN1_B, RWKV_T_LN2_W, RWKV_T_LN2_B,
  RWKV_T_X_R, RWKV_T_X_W, RWKV_T_X_K, RWKV_T_X_V, RWKV_T_X_A, RWKV_T_X_G,
  RWKV_T_W0, RWKV_T_A0, RWKV_T_V0, RWKV_T_K_K, RWKV_T_K_A, RWKV_T_R_K, RWKV_T_LNX_W, RWKV_T_LNX_B,
  RWKV_T_FFN_X_K,
  /* per-layer LoRA matrices in "out,in" layout: *1 is [R,C] (the reference's w1_t), *2 is [C,R] (w2_t) */
  RWKV_T_W1 = 40, RWKV_T_W2, RWKV_T_A1, RWKV_T_A2, RWKV_T_G1, RWKV_T_G2, RWKV_T_V1, RWKV_T_V2,
};
/* big matrices, all [N_out,K_in] row-major (ffn.value as [C,F], the checkpoint's own layout) */
enum {
  RWKV_M_ATT_R = 0, RWKV_M_ATT_K, RWKV_M_ATT_V, RWKV_M_ATT_O, RWKV_M_FFN_KEY, RWKV_M_FFN_VALUE, RWKV_M_HEAD,
};

typedef struct rwkv_hip_model rwkv_hip_model;
typedef struct rwkv_hip_session rwkv_hip_session;

int rwkv_hip_model_create(rwkv_hip_model** out, int L, int C, int H, int F, int V, int Rw, int Ra, int Rg,
                          int Rv);
int rwkv_hip_model_destroy(rwkv_hip_model* m);
/* Device pointers are borrowed: the caller owns the weights and keeps them alive. */
int rwkv_hip_model_set_tensor(rwkv_hip_model* m, int layer, int id, const void* data);
int rwkv_hip_model_set_matrix(rwkv_hip_model* m, int layer, int id, int fmt, const void* data,
                              const void* scale, const void* zp);
/* bytes of weights one decode step streams (for roofline accounting) */
int rwkv_hip_model_weight_bytes(const rwkv_hip_model* m, uint64_t* bytes);

/* A session owns a stream, the activation arena and captured decode graphs.  One session serves
 * one caller at a time; several sessions may run concurrently against one model (the reference
 * instead allocates a stream + arena per call, src/rwkv7_fast_v4.cu:1087-1096). */
int rwkv_hip_session_create(rwkv_hip_session** out, const rwkv_hip_model* m);
int rwkv_hip_session_destroy(rwkv_hip_session* s);
int rwkv_hip_session_stream(rwkv_hip_session* s, rwkv_stream_t* stream);
/* use_graph != 0: T == 1 steps replay a captured HIP graph (default on) */
int rwkv_hip_session_set_graph(rwkv_hip_session* s, int use_graph);

/* tokens_host [B,T] int64 (host); shift f16 [L,2,B,C]; wkv f32 [L,B,H,64,64] (f16 with
 * rwkv_hip_session_set_wkv_fp16); elapsed i32 [B];
 * logits f32 [B,V] for the last token of each row.  All state tensors are updated in place.
 * Returns after the work is enqueued AND complete (the reference synchronises too,
 * src/rwkv7_fast_v4.cu:1343) unless sync == 0. */
int rwkv_hip_forward(rwkv_hip_session* s, const int64_t* tokens_host, int B, int T, void* shift, void* wkv,
                     void* elapsed, void* logits, int sync);
/* Greedy decode loop kept on the device: runs `steps` decode steps at batch B, feeding each row's
 * argmax back as its next token without a host round trip; out_tokens_host [steps,B] int32.
 * first_tokens_host [B] are the tokens of step 0. */
int rwkv_hip_decode_greedy(rwkv_hip_session* s, const int64_t* first_tokens_host, int B, int steps, void* shift,
                           void* wkv, void* elapsed, void* logits, int32_t* out_tokens_host);
/* Measurement aid (no counterpart in the reference).  While a profiling mode is on, forward passes run
 * eagerly (no graph replay).  Mode 1: every weight-streaming linear launch (r/k/v, output, ffn.key,
 * ffn.value, lm_head) is bracketed by its own pair of events on the session stream.  Mode 2: a pass
 * launches ONLY those linear kernels, back to back, with one pair of events around the pass - their
 * duration does not depend on the data, and this gives the kernels' launch-to-launch time without event
 * overhead between them; state and logits hold garbage afterwards.  read_profile waits for the stream
 * and returns the number of linear launches and the summed bracketed time since the last read. */
/* Decode graphs captured so far in this process, over all sessions: a serving loop in its steady state captures
 * none (a step whose batch width, state and logits addresses have been seen replays the graph captured then). */
int rwkv_hip_graph_capture_count(int64_t* count);
int rwkv_hip_session_set_profile(rwkv_hip_session* s, int mode);
int rwkv_hip_session_read_profile(rwkv_hip_session* s, int64_t* launches, double* total_ms);
/* Decode steps of up to max_rows rows (0..12) use the row-skipping ffn.value product (CmixMode::NoFcOne / NoFcRows2
 * of the reference, include/rwkv7_fast_v4_common.hpp:198-211, whose default is 12 rows at C = 4096).  Default 4: two
 * to four rows share one walk that reads every row that is non-zero for any of them once (with a fraction z of zero
 * activations per row that is 1 - z^rows of the matrix: at the z = 0.5 of random-init weights about what the dense
 * product reads, far less with trained weights; 7.2B shape, 2 / 3 / 4 rows: 2.19 / 2.39 / 2.56 ms per step against
 * 2.61 / 2.79 / 2.82 before).  From five rows on every row walks its own rows, which pays only while rows x (1 - z)
 * stays below 1.  0 selects the dense product. */
int rwkv_hip_session_set_sparse_ffn(rwkv_hip_session* s, int max_rows);
/* on != 0: the `wkv` tensor of rwkv_hip_forward / rwkv_hip_decode_greedy is the fp16 state, f16 [L,B,H,64,64], and
 * the recurrence runs in fp16 as rwkv_hip_wkv7_f16state does (ModelBackend's use_wkv32 == false, the reference
 * server's default: src/rwkv7_fast_v4.cu:1262-1271; calls of up to 16 tokens add w0 to the decay logit unrounded,
 * longer ones round w12 + w0 to fp16 first).  Default off: fp32 state.  A state belongs to one mode. */
int rwkv_hip_session_set_wkv_fp16(rwkv_hip_session* s, int on);
/* Decode steps on the GEMV path can fold the two LayerNorm + token-shift kernels of a layer into the prologue of
 * the linear launches that consume them.  on > 0: always (where a launch with a prologue takes the rows), 0: never,
 * < 0 (the default): both LayerNorms for one or two rows of at most 4096 channels, LN2 for 5 to 8 rows of int8 / fp16
 * weights with 1024 .. 4096 channels (the few-row matrix-core launch).  One and two rows go through a kernel that
 * requests whole weight rows up front and normalises while they are in flight (two launches fewer per layer: 7.2B
 * shape, one row 2.04 -> 1.92 ms per step, 0.1B shape 0.413 -> 0.373; same formulas and rounding points as the
 * stand-alone kernels, sums associated differently); 3 to 8 rows of other shapes, when forced, through a prologue
 * that is bitwise the stand-alone kernels but slower than them from 2048 channels on.  No counterpart in the
 * reference (its fused decode kernels are cuda/rwkv7_v3a_ops.cu:1637-1798). */
int rwkv_hip_session_set_fused_ln(rwkv_hip_session* s, int on);
/* Decode steps run everything between the r/k/v projections and the output projection as one launch per layer, one
 * block per head and 1, 2 or 4 batch rows (the head's LoRA rows are loaded once per block), up to 8 rows and while
 * that launch is one round of blocks on the chip; larger batches take the row-tiled kernels of the prefill path.  rows
 * 1, 2 or 4: always the single launch, with that many rows per block where the batch is a multiple of it (else 1);
 * 0: never; < 0 (the default): by batch size.  1, 2 and 4 give the same bits; the row-tiled kernels add up the
 * LoRA rank-outs in another order (fp32 sums, then the same fp16 rounding points).  No counterpart in the reference
 * (its decode step launches the kernels of cuda/rwkv7_v3a_ops.cu:1027-1130 and cuda/rwkv7_fast_ops_fp16.cu:129-237
 * one after the other). */
int rwkv_hip_session_set_tmix_rows(rwkv_hip_session* s, int rows);
/* debugging/parity tap: device address of one of the session's activation buffers, holding what the last
 * layer of the last rwkv_hip_forward call left there.  Ids in order: x, xx, xr, xw, xk, xv, xa, xg, r, k, v,
 * v_first, w12, a12, g, hw, ha, hg, hv, k2, nkk, kka, y, y2, att, x1, ln2, mixed, act, cm (f16), then
 * r32, d32, k32, a32, b32 (f32).  Which of them a pass writes depends on its shape (decode steps fuse most
 * of them away).  No counterpart in the reference. */
int rwkv_hip_session_debug_buffer(rwkv_hip_session* s, int id, void** ptr);
/* debugging/parity tap: residual stream after every layer of the last rwkv_hip_forward call,
 * f16 [L, B*T, C], valid only if enabled before the call */
int rwkv_hip_session_set_trace(rwkv_hip_session* s, void* trace);

#ifdef __cplusplus
}
#endif
#endif
