// RWKV-7 layer graph on one GPU: model handle (borrowed weight pointers), session (stream, activation
// arena, captured decode graphs) and the forward pass for prefill chunks (T > 1) and decode steps (T == 1).
//
// Reference: run_backend_forward, src/rwkv7_fast_v4.cu:1046-1345 -- same op order, same layer-0 special
// cases (no v LoRA, v_first = v: :1171,1246-1247), same state slices (:1177-1185), logits for the last
// token of each row only (:1314-1342), elapsed += T (:1320).  Differences by design:
//   * the arena and stream live in the session instead of being allocated on every call (:1087-1096);
//   * the embedding+ln0 table stays in HBM and rows are gathered on the device (the reference gathers on
//     the host and copies, :1103-1116,1155);
//   * T == 1 steps are captured once into a HIP graph per (batch, state, logits) tuple and replayed;
//   * LN1 + the six token-shift lerps are fused for every batch size (the reference does it for B == 1).
#include <algorithm>
#include <atomic>
#include <mutex>
#include <vector>

#include <cstdlib>

#include "ops.h"

using namespace rwkv;

struct Matrix {
  int fmt = RWKV_FMT_F16;
  const void* data = nullptr;
  const half_t* scale = nullptr;
  const uint8_t* zp = nullptr;
  void* packed = nullptr;  // owned: the same codes in the MFMA-native order, for calls with >= 16 rows
  void* sparse_t = nullptr;  // owned, ffn.value only: the [F,C] copy for the one-token row-skipping product
};

struct Layer {
  const half_t* t[64] = {nullptr};
  Matrix m[6];
  void* lora_in_packed[4] = {nullptr, nullptr, nullptr, nullptr};  // owned: W1, A1, G1, V1 in the MFMA-native order
  half_t* lora_out_packed[4] = {nullptr, nullptr, nullptr, nullptr};  // owned: W2, A2, G2, V2 in the rank-out kernel's order
};

struct rwkv_hip_model {
  int L = 0, C = 0, H = 0, F = 0, V = 0, Rw = 0, Ra = 0, Rg = 0, Rv = 0;
  const half_t* emb_ln0 = nullptr;
  const half_t* ln_out_w = nullptr;
  const half_t* ln_out_b = nullptr;
  Matrix head;
  std::vector<Layer> layers;

  ~rwkv_hip_model() {
    if (head.packed) (void)hipFree(head.packed);
    for (Layer& l : layers) {
      for (Matrix& mat : l.m) {
        if (mat.packed) (void)hipFree(mat.packed);
        if (mat.sparse_t) (void)hipFree(mat.sparse_t);
      }
      for (void* q : l.lora_in_packed)
        if (q) (void)hipFree(q);
      for (half_t* q : l.lora_out_packed)
        if (q) (void)hipFree(q);
    }
  }
};

namespace {

struct GraphEntry {
  int B = 0;
  void* shift = nullptr;
  void* wkv = nullptr;
  void* elapsed = nullptr;
  void* logits = nullptr;
  hipGraphExec_t exec = nullptr;
  hipGraph_t graph = nullptr;
  uint64_t last_use = 0;
};

constexpr size_t kMaxGraphs = 8;
// Calls with at least this many rows stream the packed copy through MFMA.  Below: the weight-streaming GEMV that keeps
// whole weight rows in flight for up to 4 rows of x (decode ms per step, GEMV / streaming GEMM: 7.2B shape, int8: 3 rows
// 2.39 / 2.79, 4 rows 2.56 / 2.82; 1.5B shape: 3 rows 1.20 / 1.45, 4 rows 1.31 / 1.51, 5 rows 1.55 / 1.31; 0.1B shape,
// fp16: 3 rows 0.51 / 0.63, 4 rows 0.57 / 0.67), and from 5 to 16 rows - for int8 and fp16 weights in rows of 1024,
// 2048, 3072 or 4096 values - the same stream with the products on the matrix core (7.2B shape, int8, this / streaming
// GEMM: 5 rows 2.84 / 3.01, 8 rows 2.69 / 2.87, 16 rows 2.99 / 3.06).  RWKV_PACKED_MIN_ROWS (tuning hook) overrides
// the crossover.
constexpr int kPackedMinRows = 3;  // what gets a packed copy at all: rows too long for the GEMV (ffn.value) use it from here
constexpr int kFewRowsMax = 16;    // most rows of the few-row matrix-core launch
inline bool few_rows_on_matrix_core(const rwkv_hip_model* m) {
  if (m->layers.empty()) return false;
  const Layer& l0 = m->layers[0];
  const int mids[5] = {RWKV_M_ATT_R, RWKV_M_ATT_K, RWKV_M_ATT_V, RWKV_M_ATT_O, RWKV_M_FFN_KEY};
  for (int id : mids)
    if (!linear_rows_mfma_supported(l0.m[id].fmt, id == RWKV_M_FFN_KEY ? m->F : m->C, m->C)) return false;
  const int ranks[4] = {m->Rw, m->Ra, m->Rg, m->Rv};
  for (int r : ranks)
    if (!linear_rows_mfma_supported(RWKV_FMT_F16, r, m->C)) return false;
  return true;
}
inline int packed_min_rows(const rwkv_hip_model* m) {
  static const int forced = getenv("RWKV_PACKED_MIN_ROWS") ? atoi(getenv("RWKV_PACKED_MIN_ROWS")) : 0;
  if (forced >= kPackedMinRows) return forced;
  return few_rows_on_matrix_core(m) ? kFewRowsMax + 1 : 5;
}
// most blocks of a single-launch time-mix core beyond 8 rows (one round on the chip's compute units; us per layer at the 7.2B shape,
// this launch / the row-tiled kernels: 16 rows 14 / 17, 32 rows 25 / 24)
inline int tmix_step_max_blocks() { return device_cu_count(); }

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct Arena {
  unsigned char* base = nullptr;
  size_t cap = 0;
  size_t off = 0;
  template <typename T>
  T* take(size_t n) {
    const size_t bytes = align_up(n * sizeof(T), 256);
    T* p = reinterpret_cast<T*>(base + off);
    off += bytes;
    return p;
  }
};

struct Buffers {
  half_t *x, *xx, *xr, *xw, *xk, *xv, *xa, *xg, *r, *k, *v, *v_first, *w12, *a12, *g, *hw, *ha, *hg, *hv, *k2, *nkk,
      *kka, *y, *y2, *att, *x1, *ln2, *mixed, *act, *cm, *xf, *scratch, *shift_next;
  float *r32, *d32, *k32, *a32, *b32;
};

}  // namespace

struct rwkv_hip_session {
  const rwkv_hip_model* model = nullptr;
  hipStream_t stream = nullptr;
  Arena arena;
  int arena_B = 0, arena_T = 0;
  Buffers buf = {};
  int64_t* tokens_dev = nullptr;
  int64_t* tokens_pinned = nullptr;
  int tokens_cap = 0;
  int* argmax_dev = nullptr;
  int* history_dev = nullptr;
  size_t history_cap = 0;
  int argmax_cap = 0;
  bool use_graph = true;
  half_t* trace = nullptr;
  std::vector<GraphEntry> graphs;
  uint64_t tick = 0;
  int profile = 0;  // 0 off, 1 event pair per linear launch, 2 linear launches only with one pair per pass
  int64_t prof_launches = 0;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> prof_events;
  void* gemm_ws = nullptr;  // split-K partials of the packed GEMM
  size_t gemm_ws_bytes = 0;
  void* sparse_ws = nullptr;  // partial rows of the row-skipping ffn.value product
  size_t sparse_ws_bytes = 0;
  int sparse_ffn_rows = 4;    // decode steps of up to this many rows read only the ffn.value rows with a non-zero activation
                              // (2..4 rows share one walk over the rows that are non-zero for any of them)
  bool wkv_fp16 = false;      // the WKV state tensor is fp16 [L,B,H,64,64] (the reference's use_wkv32 == false)
  int tmix_rows = -1;         // decode steps' single-launch time-mix core: rows per block 1/2/4, 0 never, < 0 by batch
  int fused_ln = -1;          // decode steps fold LayerNorm + token shift into the linear launches: 1 always, 0 never,
                              // -1 for one row of at most 4096 channels (the row-resident GEMV hides the prologue
                              // behind its weight requests: 7.2B shape 2.04 -> 1.92 ms per step, 0.1B 0.413 -> 0.373)
};

namespace {

int model_ready(const rwkv_hip_model* m) {
  RWKV_REQUIRE(m != nullptr, "model is NULL");
  if (!m->emb_ln0 || !m->ln_out_w || !m->ln_out_b || !m->head.data) {
    set_error("model: global tensors (emb_ln0, ln_out, head) are not all set");
    return RWKV_E_STATE;
  }
  static const int vec_ids[] = {RWKV_T_LN1_W, RWKV_T_LN1_B, RWKV_T_LN2_W, RWKV_T_LN2_B, RWKV_T_X_R, RWKV_T_X_W,
                                RWKV_T_X_K,   RWKV_T_X_V,   RWKV_T_X_A,   RWKV_T_X_G,   RWKV_T_W0,  RWKV_T_A0,
                                RWKV_T_K_K,   RWKV_T_K_A,   RWKV_T_R_K,   RWKV_T_LNX_W, RWKV_T_LNX_B, RWKV_T_FFN_X_K,
                                RWKV_T_W1,    RWKV_T_W2,    RWKV_T_A1,    RWKV_T_A2,    RWKV_T_G1,  RWKV_T_G2};
  for (int l = 0; l < m->L; ++l) {
    for (int id : vec_ids) {
      if (!m->layers[l].t[id]) {
        set_error("model: layer %d tensor %d is not set", l, id);
        return RWKV_E_STATE;
      }
    }
    if (l > 0 && (!m->layers[l].t[RWKV_T_V0] || !m->layers[l].t[RWKV_T_V1] || !m->layers[l].t[RWKV_T_V2])) {
      set_error("model: layer %d value-residual tensors are not set", l);
      return RWKV_E_STATE;
    }
    for (int i = 0; i < 6; ++i) {
      if (!m->layers[l].m[i].data) {
        set_error("model: layer %d matrix %d is not set", l, i);
        return RWKV_E_STATE;
      }
    }
  }
  return RWKV_OK;
}

int ensure_arena(rwkv_hip_session* s, int B, int T) {
  const rwkv_hip_model* m = s->model;
  const size_t rows = static_cast<size_t>(B) * T;
  if (s->arena.base && B <= s->arena_B && T <= s->arena_T && B * T <= s->arena_B * s->arena_T) {
    // shapes are laid out per call below, so only capacity matters
  }
  const size_t RC = rows * m->C;
  const size_t rank_max = static_cast<size_t>(std::max(std::max(m->Rw, m->Ra), std::max(m->Rg, m->Rv)));
  size_t need = 0;
  auto add = [&](size_t n, size_t elt) { need += align_up(n * elt, 256); };
  for (int i = 0; i < 27; ++i) add(RC, 2);           // f16 [rows,C] buffers
  for (int i = 0; i < 4; ++i) add(rows * rank_max, 2);  // LoRA hidden
  add(rows * m->F, 2);                                // act
  add(static_cast<size_t>(B) * m->C, 2);              // xf
  add(static_cast<size_t>(B) * m->C, 2);              // shift_next
  add(RC, 2);                                         // scratch
  for (int i = 0; i < 5; ++i) add(RC, 4);             // fp32 WKV operands
  if (need > s->arena.cap) {
    // a larger shape invalidates captured graphs (they hold arena addresses)
    for (auto& g : s->graphs) {
      if (g.exec) (void)hipGraphExecDestroy(g.exec);
      if (g.graph) (void)hipGraphDestroy(g.graph);
    }
    s->graphs.clear();
    RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
    if (s->arena.base) RWKV_HIP_TRY(hipFree(s->arena.base));
    s->arena.base = nullptr;
    s->arena.cap = 0;
    RWKV_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&s->arena.base), need));
    s->arena.cap = need;
    s->arena_B = 0;
    s->arena_T = 0;
  }
  if (B != s->arena_B || T != s->arena_T) {
    // new layout: graphs captured for another (B,T) layout of the same arena stay valid only if the
    // layout for that B is unchanged; decode graphs are keyed by B and T == 1, and the layout below
    // depends on (B,T) only, so a (B,1) layout is always the same addresses.
    Arena& a = s->arena;
    a.off = 0;
    Buffers& b = s->buf;
    half_t** f16s[] = {&b.x, &b.xx, &b.xr, &b.xw, &b.xk, &b.xv, &b.xa, &b.xg, &b.r, &b.k, &b.v, &b.v_first, &b.w12,
                       &b.a12, &b.g, &b.k2, &b.nkk, &b.kka, &b.y, &b.y2, &b.att, &b.x1, &b.ln2, &b.mixed, &b.cm,
                       &b.scratch};
    for (half_t** p : f16s) *p = a.take<half_t>(RC);
    b.hw = a.take<half_t>(rows * rank_max);
    b.ha = a.take<half_t>(rows * rank_max);
    b.hg = a.take<half_t>(rows * rank_max);
    b.hv = a.take<half_t>(rows * rank_max);
    b.act = a.take<half_t>(rows * m->F);
    b.xf = a.take<half_t>(static_cast<size_t>(B) * m->C);
    b.shift_next = a.take<half_t>(static_cast<size_t>(B) * m->C);
    b.r32 = a.take<float>(RC);
    b.d32 = a.take<float>(RC);
    b.k32 = a.take<float>(RC);
    b.a32 = a.take<float>(RC);
    b.b32 = a.take<float>(RC);
    s->arena_B = B;
    s->arena_T = T;
  }
  // (from the smallest row count that any matrix takes through its packed copy: ffn.value's rows are too long for
  // the few-row launches)
  if (rows >= static_cast<size_t>(kPackedMinRows)) {
    const int R = static_cast<int>(rows);
    const int qkv_ns[7] = {m->C, m->C, m->C, m->Rw, m->Ra, m->Rg, m->Rv};
    size_t ws = std::max(linear_packed_multi_workspace_bytes(R, m->C, 7, qkv_ns),
                         linear_packed_multi_workspace_bytes(R, m->C, 6, qkv_ns));  // layer 0 has no v rank-in
    // (the same launch in two parts: the projections, then the rank-ins)
    ws = std::max(ws, linear_packed_multi_workspace_bytes(R, m->C, 3, qkv_ns));
    ws = std::max(ws, linear_packed_multi_workspace_bytes(R, m->C, 4, qkv_ns + 3));
    ws = std::max(ws, linear_packed_multi_workspace_bytes(R, m->C, 3, qkv_ns + 3));
    ws = std::max(ws, linear_packed_workspace_bytes(R, m->C, m->C));
    ws = std::max(ws, linear_packed_workspace_bytes(R, m->F, m->C));
    ws = std::max(ws, linear_packed_workspace_bytes(R, m->C, m->F));
    ws = std::max(ws, linear_packed_workspace_bytes(B, m->V, m->C));
    // (the column slices of ffn.value on the few-row launch: F / C planes of fp32 partial sums)
    if (R <= kFewRowsMax && m->F % m->C == 0) ws = std::max(ws, static_cast<size_t>(m->F / m->C) * R * m->C * sizeof(float));
    if (ws > s->gemm_ws_bytes) {
      for (auto& g : s->graphs) {
        if (g.exec) (void)hipGraphExecDestroy(g.exec);
        if (g.graph) (void)hipGraphDestroy(g.graph);
      }
      s->graphs.clear();
      RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
      if (s->gemm_ws) RWKV_HIP_TRY(hipFree(s->gemm_ws));
      s->gemm_ws = nullptr;
      s->gemm_ws_bytes = 0;
      RWKV_HIP_TRY(hipMalloc(&s->gemm_ws, ws));
      s->gemm_ws_bytes = ws;
    }
  }
  if (!s->sparse_ws && ffn_sparse_supported(RWKV_FMT_W8, m->C, m->F)) {
    const size_t bytes = ffn_sparse_workspace_bytes(kSparseMaxRows, m->C, m->F);
    RWKV_HIP_TRY(hipMalloc(&s->sparse_ws, bytes));
    s->sparse_ws_bytes = bytes;
  }
  if (static_cast<int>(rows) > s->tokens_cap) {
    // captured decode graphs read their tokens from the old buffer (embedding gather, token feedback)
    for (auto& g : s->graphs) {
      if (g.exec) (void)hipGraphExecDestroy(g.exec);
      if (g.graph) (void)hipGraphDestroy(g.graph);
    }
    s->graphs.clear();
    RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
    if (s->tokens_dev) RWKV_HIP_TRY(hipFree(s->tokens_dev));
    if (s->tokens_pinned) RWKV_HIP_TRY(hipHostFree(s->tokens_pinned));
    s->tokens_dev = nullptr;
    s->tokens_pinned = nullptr;
    s->tokens_cap = 0;
    RWKV_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&s->tokens_dev), rows * sizeof(int64_t)));
    RWKV_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&s->tokens_pinned), rows * sizeof(int64_t), hipHostMallocDefault));
    s->tokens_cap = static_cast<int>(rows);
  }
  return RWKV_OK;
}

// With `defer` the split-K partials of a packed call stay in the session workspace for the LayerNorm kernel that
// consumes the result (defer->partial != NULL afterwards); the workspace is rewritten by the next packed call.
int apply_matrix(const rwkv_hip_session* s, const Matrix& mat, int M, int N, int K, const half_t* x, int epilogue,
                 int out_f32, void* y, DeferredReduce* defer = nullptr, const RowCopy* copy = nullptr) {
  if (defer) *defer = DeferredReduce{};
  // (rows longer than the few-row GEMV keeps in registers go to the packed product from its smallest row count on)
  if (mat.packed && (M >= packed_min_rows(s->model) || (M >= kPackedMinRows && K > 4096))) {
    return linear_packed(s->stream, mat.fmt, M, N, K, x, mat.packed, mat.scale, mat.zp, epilogue, out_f32, y, s->gemm_ws,
                         s->gemm_ws_bytes, defer, copy);
  }
  if (copy && copy->n > 0) {
    RWKV_HIP_TRY(hipMemcpyAsync(copy->dst, copy->src, sizeof(half_t) * copy->n, hipMemcpyDeviceToDevice, s->stream));
  }
  return linear_any_m(s->stream, mat.fmt, M, N, K, x, mat.data, mat.scale, mat.zp, epilogue, out_f32, y);
}

// ffn.value of 5 to 16 rows on the few-row launch: F / C column slices of C values each, whose partial sums the
// LayerNorm kernel that consumes the result adds up and scales (7.2B shape, 8 rows: 19.4 us for the packed product).
bool sliced_value_ok(const rwkv_hip_session* s, const Matrix& mv, int rows) {
  const rwkv_hip_model* m = s->model;
  static const bool off = getenv("RWKV_SLICED_VALUE") && atoi(getenv("RWKV_SLICED_VALUE")) == 0;  // tuning hook
  static const int min_rows = getenv("RWKV_ROWS_MFMA_MIN") ? atoi(getenv("RWKV_ROWS_MFMA_MIN")) : 5;  // tuning hook
  return !off && rows >= min_rows && rows <= kFewRowsMax && m->F % m->C == 0 && m->F / m->C <= kMaxProblems &&
         (mv.fmt == RWKV_FMT_W8 || mv.fmt == RWKV_FMT_F16) && linear_rows_mfma_supported(mv.fmt, m->C, m->C) &&
         s->gemm_ws_bytes >= static_cast<size_t>(m->F / m->C) * rows * m->C * sizeof(float);
}

int sliced_value(const rwkv_hip_session* s, const Matrix& mv, int rows, const half_t* act, DeferredReduce* defer,
                 const RowCopy* copy = nullptr) {
  const rwkv_hip_model* m = s->model;
  float* ws = static_cast<float*>(s->gemm_ws);
  const int rc = linear_rows_mfma_sliced(s->stream, mv.fmt, rows, m->C, m->F, m->C, act, mv.data, ws, copy);
  if (rc != RWKV_OK) return rc;
  defer->partial = ws;
  defer->scale = mv.fmt == RWKV_FMT_W8 ? mv.scale : nullptr;
  defer->plane = static_cast<int64_t>(rows) * m->C;
  defer->splits = m->F / m->C;
  return RWKV_OK;
}

void take_deferred(LnArgs& a, const DeferredReduce& d) {
  a.res_partial = d.partial;
  a.res_scale = d.scale;
  a.res_plane = d.plane;
  a.res_splits = d.splits;
}

#define TRY(expr)                  \
  do {                             \
    const int rc__ = (expr);       \
    if (rc__ != RWKV_OK) return rc__; \
  } while (0)

// Profiling mode 1: bracket a weight-streaming linear launch with a pair of events on the session stream.
// Mode 2 only counts the launch (the pass as a whole is bracketed).
#define TRY_PROF(expr)                                              \
  do {                                                              \
    hipEvent_t e0__ = nullptr, e1__ = nullptr;                      \
    if (s->profile == 1) {                                          \
      RWKV_HIP_TRY(hipEventCreate(&e0__));                          \
      RWKV_HIP_TRY(hipEventCreate(&e1__));                          \
      RWKV_HIP_TRY(hipEventRecord(e0__, st));                       \
    }                                                               \
    const int rc__ = (expr);                                        \
    if (s->profile == 1) {                                          \
      RWKV_HIP_TRY(hipEventRecord(e1__, st));                       \
      s->prof_events.push_back(std::make_pair(e0__, e1__));         \
    }                                                               \
    if (s->profile) ++s->prof_launches;                             \
    if (rc__ != RWKV_OK) return rc__;                               \
  } while (0)

// Every launch that is not a weight-streaming linear goes through TRY_AUX: profiling mode 2 skips them, so that
// a pass consists of the linear launches alone, back to back (their duration does not depend on the data).
#define TRY_AUX(expr)                \
  do {                               \
    if (s->profile != 2) TRY(expr);  \
  } while (0)

// Enqueues the whole forward pass on the session stream.  tokens are already in s->tokens_dev.
int enqueue_forward(rwkv_hip_session* s, int B, int T, half_t* shift, void* wkv_any, int* elapsed, float* logits) {
  float* wkv = static_cast<float*>(wkv_any);            // fp32 state (the default)
  half_t* wkv16 = static_cast<half_t*>(wkv_any);        // fp16 state (session option)
  const rwkv_hip_model* m = s->model;
  hipStream_t st = s->stream;
  Buffers& b = s->buf;
  const int C = m->C, H = m->H, F = m->F, V = m->V, L = m->L;
  const int rows = B * T;
  const int64_t RC = static_cast<int64_t>(rows) * C;
  const bool step = (T == 1);
  // The weight-streaming GEMV path: below the MFMA crossover, and up to 8 rows for shapes that have no packed copy.
  bool packable = true;
  for (const Matrix& mat : m->layers[0].m) packable = packable && mat.packed != nullptr;
  for (int i = 0; i < 3; ++i) packable = packable && m->layers[0].lora_in_packed[i] != nullptr;
  const bool small = rows < packed_min_rows(m) || (rows <= 8 && !packable);
  hipEvent_t pass_begin = nullptr;
  if (s->profile == 2) {
    RWKV_HIP_TRY(hipEventCreate(&pass_begin));
    RWKV_HIP_TRY(hipEventRecord(pass_begin, st));
  }
  // The single-launch time-mix core loads a head's LoRA rows once per block, for 1, 2 or 4 batch rows.  It is used
  // up to 8 rows and while the launch is one round of blocks on the chip; beyond that the row-tiled kernels of the
  // prefill path (LoRA rank-outs on the matrix core, the recurrence at full memory rate) are faster.  The fp16 state and
  // batches that are no multiple of 2 or 4 keep one row per block.
  int tmix_rows = 0;
  if (step) {
    if (s->tmix_rows > 0) {
      tmix_rows = (B % s->tmix_rows == 0 && !s->wkv_fp16) ? s->tmix_rows : 1;
    } else if (s->tmix_rows < 0) {
      const int rpb = tmix_step_rows_per_block(B, H, s->wkv_fp16);
      if (rows <= 8 || B * H / rpb <= tmix_step_max_blocks()) tmix_rows = rpb;
    }
  }
  const bool fused_tmix = tmix_rows > 0;
  // Decode steps on the GEMV path can fold both LayerNorm + token-shift kernels of a layer into the prologue of the
  // linear launch that consumes them (r/k/v + LoRA rank-ins; ffn.key): by default for one row of up to 4096
  // channels.  The residual-stream tap needs the stand-alone kernels.
  const bool want_ln_in_linear = s->fused_ln > 0 || (s->fused_ln < 0 && rows <= linear_ln_prologue_max_rows(C));
  // (the shift row that the prologue leaves for later is stored by the single-launch time-mix core)
  // (forced on, it also takes the rows that a launch with a prologue exists for: 5 to 8 on the few-row matrix-core
  // launch, up to 8 through the tiled GEMV while the rows fit its LDS)
  const bool ln_in_linear = want_ln_in_linear && step && small && !s->trace && fused_tmix &&
                            (rows <= linear_ln_prologue_max_rows(C) ||
                             (linear_ln_prologue_rows_ok(m->layers[0].m[RWKV_M_ATT_R].fmt, rows, C, C) &&
                              linear_ln_prologue_rows_ok(m->layers[0].m[RWKV_M_FFN_KEY].fmt, rows, F, C)) ||
                             (rows <= 8 && static_cast<size_t>(rows) * C * 2 + static_cast<size_t>(C) * 4 <= 49152));
  // 5 to 8 rows on the few-row matrix-core launch: LN2 (+ its token shift) folds into the ffn.key launch.  LN1 stays a
  // launch of its own there: it sums the split-K partials of the packed ffn.value product, which would otherwise
  // cost the reduce launch that the folded LayerNorm saves.
  const bool ln2_in_linear =
      ln_in_linear || (s->fused_ln != 0 && step && small && !s->trace && rows >= 5 &&
                       linear_ln_prologue_rows_ok(m->layers[0].m[RWKV_M_FFN_KEY].fmt, rows, F, C));
  // One row: the gate rank-out of the time-mix core (more than half of its bytes) runs in blocks of its own and the
  // output projection's launch applies the gate while it stages x.
  const bool gate_split = fused_tmix && rows == 1 && C <= 4096 && !s->trace;

  // Decode steps of a few rows (one by default) read, per row, only the ffn.value rows whose relu^2 activation is
  // non-zero (int8 or fp16 weights).
  const bool sparse_value = step && rows <= s->sparse_ffn_rows && s->sparse_ws != nullptr;

  // Prefill chunks of up to 256 rows: residual add + LayerNorm + token shift as one launch per LayerNorm (the block
  // of a row also normalises the previous row).  The new shift rows come out in a buffer of their own - the blocks
  // of the first tokens still read the old ones - and the next packed launch moves them into the state.  The block
  // reads the residual and the split-K partials of two rows, which from a few hundred rows on costs more than the
  // launch it saves (prefill of a 4096-token prompt in chunks of 128: 22.6 -> 23.2 k tok/s at batch 1, 54.2 ->
  // 53.4 k at batch 16).  RWKV_SEQ_LN=0 (tuning hook) switches it off.
  static const bool seq_ln_on = !(getenv("RWKV_SEQ_LN") && atoi(getenv("RWKV_SEQ_LN")) == 0);
  const bool seq_fused = seq_ln_on && !step && !s->trace && C <= 4096 && rows >= packed_min_rows(m) && rows <= 256;
  RowCopy pending;  // shift rows waiting to be moved
  auto flush_pending = [&]() -> int {
    if (pending.n > 0) {
      RWKV_HIP_TRY(hipMemcpyAsync(pending.dst, pending.src, sizeof(half_t) * pending.n, hipMemcpyDeviceToDevice, st));
      pending = RowCopy{};
    }
    return RWKV_OK;
  };

  auto mix6_args = [&](const Layer& w, LnArgs& a) {
    const int ids[6] = {RWKV_T_X_R, RWKV_T_X_W, RWKV_T_X_K, RWKV_T_X_V, RWKV_T_X_A, RWKV_T_X_G};
    half_t* outs[6] = {b.xr, b.xw, b.xk, b.xv, b.xa, b.xg};
    for (int i = 0; i < 6; ++i) {
      a.mu[i] = w.t[ids[i]];
      a.out[i] = outs[i];
    }
    a.n_mix = 6;
  };

  if (ln_in_linear) {
    // nothing here: layer 0's r/k/v launch gathers the embedding rows itself
  } else if (step) {
    // embedding gather + LN1(layer 0) + six lerps + shift0 write in one kernel
    LnArgs a = {};
    a.x = m->emb_ln0; a.tokens = s->tokens_dev; a.x_out = b.x;
    a.w = m->layers[0].t[RWKV_T_LN1_W]; a.b = m->layers[0].t[RWKV_T_LN1_B];
    a.shift = shift; a.C = C; a.T = 1; a.eps = kLnEps;
    mix6_args(m->layers[0], a);
    TRY_AUX(ln_launch(st, kLnMix, rows, a));
  } else {
    TRY_AUX(embed_gather_launch(st, rows, C, s->tokens_dev, m->emb_ln0, b.x));
    LnArgs a = {};
    a.x = b.x; a.w = m->layers[0].t[RWKV_T_LN1_W]; a.b = m->layers[0].t[RWKV_T_LN1_B]; a.y = b.xx;
    a.C = C; a.T = 1; a.eps = kLnEps;
    TRY_AUX(ln_launch(st, kLn, rows, a));
  }

  for (int l = 0; l < L; ++l) {
    const Layer& w = m->layers[l];
    half_t* shift0 = shift + static_cast<int64_t>(l) * 2 * B * C;
    half_t* shift1 = shift0 + static_cast<int64_t>(B) * C;
    float* S = wkv + static_cast<int64_t>(l) * B * H * kHead * kHead;
    half_t* S16 = wkv16 + static_cast<int64_t>(l) * B * H * kHead * kHead;
    half_t* v_cur = (l == 0) ? b.v_first : b.v;  // layer 0 writes v straight into v_first

    if (!step && pending.n == 0) {  // (with rows pending, the previous layer's last launch has mixed already)
      MixArgs a = {};
      a.x = b.xx; a.shift = shift0; a.B = B; a.T = T; a.C = C; a.n_mix = 6;
      const int ids[6] = {RWKV_T_X_R, RWKV_T_X_W, RWKV_T_X_K, RWKV_T_X_V, RWKV_T_X_A, RWKV_T_X_G};
      half_t* outs[6] = {b.xr, b.xw, b.xk, b.xv, b.xa, b.xg};
      for (int i = 0; i < 6; ++i) {
        a.mu[i] = w.t[ids[i]];
        a.out[i] = outs[i];
      }
      TRY_AUX(token_shift_mix_launch(st, a));
    }

    // r, k, v projections and the LoRA rank-ins (w, a, g and, past layer 0, v)
    {
      const int n_lora = (l == 0) ? 3 : 4;
      const int w1_ids[4] = {RWKV_T_W1, RWKV_T_A1, RWKV_T_G1, RWKV_T_V1};
      const int ranks[4] = {m->Rw, m->Ra, m->Rg, m->Rv};
      const half_t* lx[4] = {b.xw, b.xa, b.xg, b.xv};
      half_t* lh[4] = {b.hw, b.ha, b.hg, b.hv};
      const int mids[3] = {RWKV_M_ATT_R, RWKV_M_ATT_K, RWKV_M_ATT_V};
      const half_t* xs[3] = {b.xr, b.xk, b.xv};
      half_t* ys[3] = {b.r, b.k, v_cur};
      if (small) {
        TRY(flush_pending());
        // one launch: three big matrices (any format) + the rank-in matrices (fp16), all with K = C
        // The rank-in blocks come first: with fp16 weights against int8 they are the longest of the launch, and
        // blocks start in id order - at the end they would run on alone.
        LinearProblem p[7];
        for (int i = 0; i < n_lora; ++i) {
          p[i].w = w.t[w1_ids[i]]; p[i].scale = nullptr; p[i].zp = nullptr;
          p[i].x = lx[i]; p[i].y = lh[i]; p[i].N = ranks[i]; p[i].fmt = RWKV_FMT_F16;
        }
        for (int i = 0; i < 3; ++i) {
          LinearProblem& q = p[n_lora + i];
          q.w = w.m[mids[i]].data; q.scale = w.m[mids[i]].scale; q.zp = w.m[mids[i]].zp;
          q.x = xs[i]; q.y = ys[i]; q.N = C; q.fmt = w.m[mids[i]].fmt;
        }
        if (ln_in_linear) {
          const int lora_mu[4] = {RWKV_T_X_W, RWKV_T_X_A, RWKV_T_X_G, RWKV_T_X_V};
          const int dense_mu[3] = {RWKV_T_X_R, RWKV_T_X_K, RWKV_T_X_V};
          for (int i = 0; i < 3 + n_lora; ++i) {
            p[i].x = nullptr;
            p[i].mu = w.t[i < n_lora ? lora_mu[i] : dense_mu[i - n_lora]];
          }
          LnPrologue ln;
          ln.w = w.t[RWKV_T_LN1_W]; ln.b = w.t[RWKV_T_LN1_B]; ln.shift = shift0; ln.x_out = b.x; ln.ln_out = b.xx;
          ln.eps = kLnEps;
          if (l == 0) {
            ln.mode = 2; ln.x = m->emb_ln0; ln.tokens = s->tokens_dev;
          } else {
            ln.mode = 1; ln.x = b.x1; ln.res = b.cm;
          }
          TRY_PROF(linear_small_m(st, rows, C, 3 + n_lora, p, RWKV_EPI_NONE, 0, &ln));
        } else {
          TRY_PROF(linear_small_m(st, rows, C, 3 + n_lora, p, RWKV_EPI_NONE, 0));
        }
      } else {
        bool all_packed = rows >= packed_min_rows(m);
        for (int i = 0; i < 3; ++i) all_packed = all_packed && w.m[mids[i]].packed != nullptr;
        for (int i = 0; i < n_lora; ++i) all_packed = all_packed && w.lora_in_packed[i] != nullptr;
        if (all_packed) {
          // one streaming-GEMM launch (+ one split-K reduce) for the three projections and the rank-ins
          PackedProblem p[7];
          for (int i = 0; i < 3; ++i)
            p[i] = PackedProblem{w.m[mids[i]].packed, w.m[mids[i]].scale, w.m[mids[i]].zp, xs[i], ys[i], C, w.m[mids[i]].fmt};
          for (int i = 0; i < n_lora; ++i)
            p[3 + i] = PackedProblem{w.lora_in_packed[i], nullptr, nullptr, lx[i], lh[i], ranks[i], RWKV_FMT_F16};
          // Where a launch of int8 problems only has a tile of its own (several wavefronts per SIMD), three int8
          // projections go without the fp16 rank-ins, which follow in a launch of their own.
          bool w8_only = linear_packed_int8_tile(rows, C);
          for (int i = 0; i < 3; ++i) w8_only = w8_only && p[i].fmt == RWKV_FMT_W8;
          const RowCopy moved = pending;
          pending = RowCopy{};
          if (w8_only) {
            TRY_PROF(linear_packed_multi(st, rows, C, 3, p, RWKV_EPI_NONE, 0, s->gemm_ws, s->gemm_ws_bytes, nullptr, &moved));
            TRY_PROF(linear_packed_multi(st, rows, C, n_lora, p + 3, RWKV_EPI_NONE, 0, s->gemm_ws, s->gemm_ws_bytes));
          } else {
            TRY_PROF(linear_packed_multi(st, rows, C, 3 + n_lora, p, RWKV_EPI_NONE, 0, s->gemm_ws, s->gemm_ws_bytes, nullptr,
                                         &moved));
          }
        } else {
          TRY(flush_pending());
          for (int i = 0; i < 3; ++i) TRY_PROF(apply_matrix(s, w.m[mids[i]], rows, C, C, xs[i], RWKV_EPI_NONE, 0, ys[i]));
          for (int i = 0; i < n_lora; ++i)
            TRY_AUX(linear_any_m(st, RWKV_FMT_F16, rows, ranks[i], C, lx[i], w.t[w1_ids[i]], nullptr, nullptr, RWKV_EPI_NONE,
                             0, lh[i]));
        }
      }
    }

    if (fused_tmix) {
      // the whole time-mix core of a decode step in one launch per layer
      TmixStepArgs p = {};
      p.B = B; p.H = H; p.C = C; p.Rw = m->Rw; p.Ra = m->Ra; p.Rg = m->Rg; p.Rv = m->Rv;
      p.hw = b.hw; p.ha = b.ha; p.hg = b.hg; p.hv = (l > 0) ? b.hv : nullptr;
      p.w2 = w.t[RWKV_T_W2]; p.a2 = w.t[RWKV_T_A2]; p.g2 = w.t[RWKV_T_G2]; p.v2 = w.t[RWKV_T_V2];
      p.w0 = w.t[RWKV_T_W0]; p.a0 = w.t[RWKV_T_A0]; p.v0 = w.t[RWKV_T_V0]; p.k_k = w.t[RWKV_T_K_K];
      p.k_a = w.t[RWKV_T_K_A]; p.r_k = w.t[RWKV_T_R_K]; p.lnx_w = w.t[RWKV_T_LNX_W]; p.lnx_b = w.t[RWKV_T_LNX_B];
      p.r = b.r; p.k = b.k; p.v = v_cur; p.v_first = b.v_first; p.v_first_out = nullptr;
      p.y2 = b.y2;
      if (s->wkv_fp16) {
        p.state16 = S16; p.elapsed = elapsed;
      } else {
        p.state = S;
      }
      if (ln_in_linear) {
        p.shift_src = b.xx; p.shift_dst = shift0;
      }
      if (gate_split) {  // the g rank-out in blocks of its own; the output projection applies the gate
        p.y2_pre = b.r32; p.gate_out = b.g;
      }
      p.rows_per_block = gate_split ? 1 : tmix_rows;
      TRY_AUX(tmix_step_launch(st, p));
    } else {
      // LoRA rank-out (+ activation, + v-residual gate)
      {
        LoraOutMultiArgs a = {};
        a.M = rows; a.C = C; a.n = (l > 0) ? 4 : 3;
        a.p[0].h = b.hw; a.p[0].w2 = w.t[RWKV_T_W2]; a.p[0].R = m->Rw; a.p[0].act = RWKV_ACT_TANH; a.p[0].out = b.w12;
        a.p[1].h = b.ha; a.p[1].w2 = w.t[RWKV_T_A2]; a.p[1].R = m->Ra; a.p[1].act = RWKV_ACT_NONE; a.p[1].out = b.a12;
        a.p[2].h = b.hg; a.p[2].w2 = w.t[RWKV_T_G2]; a.p[2].R = m->Rg; a.p[2].act = RWKV_ACT_SIGMOID; a.p[2].out = b.g;
        for (int i = 0; i < 3; ++i) a.p[i].w2p = w.lora_out_packed[i];
        if (l > 0) {
          LoraOutProblem& pv = a.p[3];
          pv.h = b.hv; pv.w2 = w.t[RWKV_T_V2]; pv.w2p = w.lora_out_packed[3]; pv.R = m->Rv; pv.act = RWKV_ACT_NONE;
          pv.bias = w.t[RWKV_T_V0];
          pv.vres = 1; pv.v = b.v; pv.v_first = b.v_first; pv.out = b.xv;  // xv is free after the projections
          v_cur = b.xv;
        }
        TRY_AUX(lora_out_multi(st, a));
      }

      if (s->wkv_fp16) {
        // fp16 state (src/rwkv7_fast_v4.cu:1262-1271): kk / a-gate in fp16, the fp16 recurrence, GroupNorm / bonus / gate.
        // Calls of up to 16 tokens add w0 to the decay logit inside the recurrence, unrounded; longer ones round
        // w12 + w0 to fp16 first, as the reference does.
        if (step && !s->trace) {
          // a decode step: the three in one launch (same bits), the state moved in coalesced 1 KB requests
          Tmix16RowsArgs f = {};
          f.rows_heads = static_cast<int64_t>(rows) * H; f.H = H; f.state = S16; f.elapsed = elapsed;
          f.r = b.r; f.k = b.k; f.v = v_cur; f.w12 = b.w12; f.a12 = b.a12; f.g = b.g;
          f.k_k = w.t[RWKV_T_K_K]; f.a0 = w.t[RWKV_T_A0]; f.k_a = w.t[RWKV_T_K_A]; f.w0 = w.t[RWKV_T_W0];
          f.r_k = w.t[RWKV_T_R_K]; f.lnx_w = w.t[RWKV_T_LNX_W]; f.lnx_b = w.t[RWKV_T_LNX_B]; f.y2 = b.y2;
          TRY_AUX(tmix16_rows_launch(st, f));
        } else {
        KkArgs p = {};
        p.k = b.k; p.k_k = w.t[RWKV_T_K_K]; p.a0 = w.t[RWKV_T_A0]; p.a12 = b.a12; p.k_a = w.t[RWKV_T_K_A];
        p.new_k = b.k2; p.neg_kk = b.nkk; p.kka = b.kka;
        p.rows_heads = static_cast<int64_t>(rows) * H; p.H = H;
        const half_t* w_in = b.w12;
        const half_t* w0 = w.t[RWKV_T_W0];
        if (T > 16) {  // w12 + w0 rounded to fp16 first: the same pass writes it
          p.w12 = b.w12; p.w0 = w.t[RWKV_T_W0]; p.w_sum16 = b.scratch;
          w_in = b.scratch;
          w0 = nullptr;
        }
        TRY_AUX(kk_a_gate_launch(st, p));
        TRY_AUX(wkv7_f16state_launch(st, B, T, C, H, S16, b.r, w_in, w0, b.k2, v_cur, b.nkk, b.kka, b.y, elapsed));
        TRY_AUX(lnx_launch(st, static_cast<int64_t>(rows) * H, H, b.y, b.r, b.k2, v_cur, w.t[RWKV_T_R_K], w.t[RWKV_T_LNX_W],
                           w.t[RWKV_T_LNX_B], b.g, b.y2));
        }
      } else if (!s->trace && tmix_seq_whole_heads(B, T, H)) {
        // kk normalise / a-gate / decay, the WKV recurrence and GroupNorm / bonus / gate in one launch
        TmixSeqArgs fa;
        fa.r = b.r; fa.k = b.k; fa.a12 = b.a12; fa.w12 = b.w12; fa.g = b.g;
        fa.k_k = w.t[RWKV_T_K_K]; fa.a0 = w.t[RWKV_T_A0]; fa.k_a = w.t[RWKV_T_K_A]; fa.w0 = w.t[RWKV_T_W0];
        fa.r_k = w.t[RWKV_T_R_K]; fa.lnx_w = w.t[RWKV_T_LNX_W]; fa.lnx_b = w.t[RWKV_T_LNX_B];
        TRY_AUX(tmix_seq_launch(st, B, T, C, H, S, fa, v_cur, b.y2));
      } else {
        // with the residual-stream tap on, or few heads in flight: the three stand-alone kernels (same arithmetic,
        // bitwise the same)
        KkArgs p = {};
        p.k = b.k; p.k_k = w.t[RWKV_T_K_K]; p.a0 = w.t[RWKV_T_A0]; p.a12 = b.a12; p.k_a = w.t[RWKV_T_K_A];
        p.new_k = b.k2; p.neg_kk = nullptr; p.kka = nullptr;
        p.w12 = b.w12; p.w0 = w.t[RWKV_T_W0]; p.r = b.r;
        p.k32 = b.k32; p.a32 = b.a32; p.b32 = b.b32; p.d32 = b.d32; p.r32 = b.r32;
        p.rows_heads = static_cast<int64_t>(rows) * H; p.H = H;
        TRY_AUX(kk_a_gate_launch(st, p));
        TRY_AUX(wkv7_seq_f16_launch(st, B, T, C, H, S, b.r32, b.d32, b.k32, b.a32, b.b32, static_cast<int64_t>(T) * C, v_cur,
                                b.y, static_cast<int64_t>(T) * C));
        TRY_AUX(lnx_launch(st, static_cast<int64_t>(rows) * H, H, b.y, b.r, b.k2, v_cur, w.t[RWKV_T_R_K], w.t[RWKV_T_LNX_W],
                       w.t[RWKV_T_LNX_B], b.g, b.y2));
      }
    }
    // From 16 rows on (the streaming GEMM) the LayerNorm kernels that consume the output projection and
    // ffn.value sum the split-K partials themselves instead of a reduce launch; att / cm then stay unwritten.
    const bool defer_ok = !s->trace && !ln_in_linear;
    DeferredReduce att_partial;
    if (gate_split) {
      const Matrix& mo = w.m[RWKV_M_ATT_O];
      LinearProblem po = {mo.data, mo.scale, mo.zp, nullptr, b.att, C, mo.fmt, nullptr};
      po.x_f32 = b.r32;
      po.x_gate = b.g;
      TRY_PROF(linear_small_m(st, 1, C, 1, &po, RWKV_EPI_NONE, 0));
    } else {
      TRY_PROF(apply_matrix(s, w.m[RWKV_M_ATT_O], rows, C, C, b.y2, RWKV_EPI_NONE, 0, b.att, defer_ok ? &att_partial : nullptr));
    }

    // residual add + LN2 + channel-mix token shift
    if (ln2_in_linear) {
      // folded into the ffn.key launch below
    } else if (step) {
      LnArgs a = {};
      a.x = b.x; a.res = b.att; a.w = w.t[RWKV_T_LN2_W]; a.b = w.t[RWKV_T_LN2_B]; a.x_out = b.x1; a.shift = shift1;
      a.mu[0] = w.t[RWKV_T_FFN_X_K]; a.out[0] = b.mixed; a.n_mix = 1; a.C = C; a.T = 1; a.eps = kLnEps;
      take_deferred(a, att_partial);
      TRY_AUX(ln_launch(st, kAddLnMix, rows, a));
    } else if (seq_fused) {
      LnArgs a = {};
      a.x = b.x; a.res = b.att; a.w = w.t[RWKV_T_LN2_W]; a.b = w.t[RWKV_T_LN2_B]; a.x_out = b.x1; a.y = b.ln2;
      a.shift = shift1; a.shift_next = b.shift_next;
      a.mu[0] = w.t[RWKV_T_FFN_X_K]; a.out[0] = b.mixed; a.n_mix = 1; a.C = C; a.T = T; a.eps = kLnEps;
      take_deferred(a, att_partial);
      TRY_AUX(ln_launch(st, kAddLnMixSeq, rows, a));
      pending.src = b.shift_next; pending.dst = shift1; pending.n = B * C;
    } else {
      LnArgs a = {};
      a.x = b.x; a.res = b.att; a.w = w.t[RWKV_T_LN2_W]; a.b = w.t[RWKV_T_LN2_B]; a.x_out = b.x1; a.y = b.ln2;
      a.C = C; a.T = 1; a.eps = kLnEps;
      take_deferred(a, att_partial);
      TRY_AUX(ln_launch(st, kAddLn, rows, a));
      MixArgs mx = {};
      mx.x = b.ln2; mx.shift = shift1; mx.B = B; mx.T = T; mx.C = C; mx.n_mix = 1;
      mx.mu[0] = w.t[RWKV_T_FFN_X_K]; mx.out[0] = b.mixed;
      TRY_AUX(token_shift_mix_launch(st, mx));
    }

    // channel mix
    DeferredReduce cm_partial;
    if (ln2_in_linear) {
      const Matrix& mk = w.m[RWKV_M_FFN_KEY];
      LinearProblem pk = {mk.data, mk.scale, mk.zp, nullptr, b.act, F, mk.fmt, w.t[RWKV_T_FFN_X_K]};
      LnPrologue ln;
      ln.mode = 1; ln.x = b.x; ln.res = b.att; ln.w = w.t[RWKV_T_LN2_W]; ln.b = w.t[RWKV_T_LN2_B];
      ln.shift = shift1; ln.x_out = b.x1; ln.ln_out = b.ln2; ln.eps = kLnEps;
      TRY_PROF(linear_small_m(st, rows, C, 1, &pk, RWKV_EPI_RELU_SQUARE, 0, &ln));
      // the ffn.value launch also moves the LN2 output kept above into the channel-mix shift row of the state
      const Matrix& mv = w.m[RWKV_M_FFN_VALUE];
      RowCopy cp;
      cp.src = b.ln2; cp.dst = shift1; cp.n = rows * C;
      if (sparse_value && mv.sparse_t) {
        TRY_AUX(ffn_sparse_launch(st, mv.fmt, rows, C, F, 1, b.act, mv.sparse_t, mv.scale, s->sparse_ws, s->sparse_ws_bytes, b.cm,
                                  &cp, true));
      } else if (defer_ok && sliced_value_ok(s, mv, rows)) {
        TRY_PROF(sliced_value(s, mv, rows, b.act, &cm_partial, &cp));
      } else if (rows > 8 || (mv.packed && rows >= kPackedMinRows)) {
        // (rows too long for the few-row launches: the packed product, whose first block moves the row too)
        TRY_PROF(apply_matrix(s, mv, rows, C, F, b.act, RWKV_EPI_NONE, 0, b.cm, defer_ok ? &cm_partial : nullptr, &cp));
      } else {
        LinearProblem pv = {mv.data, mv.scale, mv.zp, b.act, b.cm, C, mv.fmt, nullptr};
        TRY_PROF(linear_small_m(st, rows, F, 1, &pv, RWKV_EPI_NONE, 0, nullptr, &cp));
      }
    } else {
      const RowCopy moved = pending;
      pending = RowCopy{};
      TRY_PROF(apply_matrix(s, w.m[RWKV_M_FFN_KEY], rows, F, C, b.mixed, RWKV_EPI_RELU_SQUARE, 0, b.act, nullptr, &moved));
      const Matrix& mv = w.m[RWKV_M_FFN_VALUE];
      if (sparse_value && mv.sparse_t) {
        TRY_AUX(ffn_sparse_launch(st, mv.fmt, rows, C, F, 1, b.act, mv.sparse_t, mv.scale, s->sparse_ws, s->sparse_ws_bytes, b.cm,
                                  nullptr, true));
      } else if (defer_ok && step && sliced_value_ok(s, mv, rows)) {
        TRY_PROF(sliced_value(s, mv, rows, b.act, &cm_partial));
      } else {
        TRY_PROF(apply_matrix(s, mv, rows, C, F, b.act, RWKV_EPI_NONE, 0, b.cm, defer_ok ? &cm_partial : nullptr));
      }
    }

    // residual add + next layer's LN1 (+ lerps), or the final LN on the last token of each row
    if (l + 1 < L && ln_in_linear) {
      // the next layer's r/k/v launch adds the residual and normalises
    } else if (l + 1 < L) {
      const Layer& nx = m->layers[l + 1];
      LnArgs a = {};
      a.x = b.x1; a.res = b.cm; a.w = nx.t[RWKV_T_LN1_W]; a.b = nx.t[RWKV_T_LN1_B]; a.x_out = b.x;
      a.C = C; a.T = 1; a.eps = kLnEps;
      take_deferred(a, cm_partial);
      if (step) {
        a.shift = shift + static_cast<int64_t>(l + 1) * 2 * B * C;
        mix6_args(nx, a);
        TRY_AUX(ln_launch(st, kAddLnMix, rows, a));
      } else if (seq_fused) {
        a.shift = shift + static_cast<int64_t>(l + 1) * 2 * B * C;
        a.shift_next = b.shift_next;
        a.y = b.xx;
        a.T = T;
        mix6_args(nx, a);
        TRY_AUX(ln_launch(st, kAddLnMixSeq, rows, a));
        pending.src = b.shift_next; pending.dst = a.shift; pending.n = B * C;
      } else {
        a.y = b.xx;
        TRY_AUX(ln_launch(st, kAddLn, rows, a));
      }
    } else {
      LnArgs a = {};
      a.x = b.x1; a.res = b.cm; a.w = m->ln_out_w; a.b = m->ln_out_b; a.y = b.xf; a.C = C; a.T = T; a.eps = kLnEps;
      take_deferred(a, cm_partial);
      TRY_AUX(ln_launch(st, kAddLastLn, B, a));
      if (s->trace) {
        LnArgs t = {};
        t.x = b.x1; t.res = b.cm; t.w = m->ln_out_w; t.b = m->ln_out_b; t.x_out = b.x; t.y = b.scratch;
        t.C = C; t.T = 1; t.eps = kLnEps;
        TRY_AUX(ln_launch(st, kAddLn, rows, t));
      }
    }
    if (s->trace) {
      RWKV_HIP_TRY(hipMemcpyAsync(s->trace + static_cast<int64_t>(l) * RC, b.x, sizeof(half_t) * RC,
                                  hipMemcpyDeviceToDevice, st));
    }
  }

  TRY(flush_pending());
  TRY_AUX(advance_launch(st, B, T, elapsed));
  TRY_PROF(apply_matrix(s, m->head, B, V, C, b.xf, RWKV_EPI_NONE, 1, logits));
  if (pass_begin) {
    hipEvent_t pass_end = nullptr;
    RWKV_HIP_TRY(hipEventCreate(&pass_end));
    RWKV_HIP_TRY(hipEventRecord(pass_end, st));
    s->prof_events.push_back(std::make_pair(pass_begin, pass_end));
  }
  return RWKV_OK;
}

std::atomic<int64_t> g_graph_captures{0};  // decode graphs captured in this process (all sessions)

GraphEntry* find_graph(rwkv_hip_session* s, int B, void* shift, void* wkv, void* elapsed, void* logits) {
  for (auto& g : s->graphs) {
    if (g.B == B && g.shift == shift && g.wkv == wkv && g.elapsed == elapsed && g.logits == logits) return &g;
  }
  return nullptr;
}

// T == 1 step through a captured graph (captures on first use of this (B, state, logits) tuple).
int run_step(rwkv_hip_session* s, int B, half_t* shift, void* wkv, int* elapsed, float* logits) {
  if (!s->use_graph || s->trace || s->profile) return enqueue_forward(s, B, 1, shift, wkv, elapsed, logits);
  GraphEntry* g = find_graph(s, B, shift, wkv, elapsed, logits);
  if (!g) {
    if (s->graphs.size() >= kMaxGraphs) {
      auto victim = std::min_element(s->graphs.begin(), s->graphs.end(),
                                     [](const GraphEntry& x, const GraphEntry& y) { return x.last_use < y.last_use; });
      RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
      if (victim->exec) (void)hipGraphExecDestroy(victim->exec);
      if (victim->graph) (void)hipGraphDestroy(victim->graph);
      s->graphs.erase(victim);
    }
    GraphEntry e;
    e.B = B; e.shift = shift; e.wkv = wkv; e.elapsed = elapsed; e.logits = logits;
    RWKV_HIP_TRY(hipStreamBeginCapture(s->stream, hipStreamCaptureModeThreadLocal));
    const int rc = enqueue_forward(s, B, 1, shift, wkv, elapsed, logits);
    hipGraph_t graph = nullptr;
    const hipError_t end = hipStreamEndCapture(s->stream, &graph);
    if (rc != RWKV_OK) {
      if (graph) (void)hipGraphDestroy(graph);
      return rc;
    }
    if (end != hipSuccess) {
      set_error("hipStreamEndCapture failed: %s", hipGetErrorString(end));
      return RWKV_E_RUNTIME;
    }
    e.graph = graph;
    RWKV_HIP_TRY(hipGraphInstantiate(&e.exec, graph, nullptr, nullptr, 0));
    g_graph_captures.fetch_add(1, std::memory_order_relaxed);
    s->graphs.push_back(e);
    g = &s->graphs.back();
  }
  g->last_use = ++s->tick;
  RWKV_HIP_TRY(hipGraphLaunch(g->exec, s->stream));
  return RWKV_OK;
}

int check_forward_args(const rwkv_hip_session* s, int B, int T, const void* shift, const void* wkv, const void* elapsed,
                       const void* logits) {
  RWKV_REQUIRE(s != nullptr, "session is NULL");
  RWKV_REQUIRE(B > 0, "token_batches must not be empty");         // src/rwkv7_fast_v4.cu:1054-1056
  RWKV_REQUIRE(T > 0, "token batch length must be positive");     // :1065-1067
  RWKV_REQUIRE(shift && wkv && elapsed && logits, "forward: NULL state or logits tensor");
  return model_ready(s->model);
}

}  // namespace

extern "C" {

int rwkv_hip_model_create(rwkv_hip_model** out, int L, int C, int H, int F, int V, int Rw, int Ra, int Rg, int Rv) {
  RWKV_REQUIRE(out != nullptr, "model out is NULL");
  *out = nullptr;
  RWKV_REQUIRE(L > 0 && H > 0 && F > 0 && V > 0, "model: L, H, F, V must be positive");
  RWKV_REQUIRE(C == H * kHead, "C must equal H*N with head size 64 (C=%d, H=%d)", C, H);  // rwkv7_fast_v4_common.hpp:285-286
  RWKV_REQUIRE(C % 32 == 0 && F % 32 == 0 && V % 4 == 0, "model: C, F must be multiples of 32 and V of 4");
  const int ranks[4] = {Rw, Ra, Rg, Rv};
  for (int r : ranks)
    RWKV_REQUIRE(r > 0 && r % 8 == 0 && r <= 512, "lowrank exceeds arena max or is not a multiple of 8 (%d)", r);  // :1172-1175
  rwkv_hip_model* m = new (std::nothrow) rwkv_hip_model();
  if (!m) {
    set_error("model: out of host memory");
    return RWKV_E_NOMEM;
  }
  m->L = L; m->C = C; m->H = H; m->F = F; m->V = V; m->Rw = Rw; m->Ra = Ra; m->Rg = Rg; m->Rv = Rv;
  m->layers.resize(L);
  *out = m;
  return RWKV_OK;
}

int rwkv_hip_model_destroy(rwkv_hip_model* m) {
  delete m;
  return RWKV_OK;
}

int rwkv_hip_model_set_tensor(rwkv_hip_model* m, int layer, int id, const void* data) {
  RWKV_REQUIRE(m && data, "set_tensor: NULL argument");
  const half_t* p = static_cast<const half_t*>(data);
  if (layer < 0) {
    switch (id) {
      case RWKV_T_EMB_LN0: m->emb_ln0 = p; return RWKV_OK;
      case RWKV_T_LN_OUT_W: m->ln_out_w = p; return RWKV_OK;
      case RWKV_T_LN_OUT_B: m->ln_out_b = p; return RWKV_OK;
      default: break;
    }
    set_error("set_tensor: unknown global tensor id %d", id);
    return RWKV_E_INVALID;
  }
  RWKV_REQUIRE(layer < m->L, "set_tensor: layer %d out of range", layer);
  RWKV_REQUIRE((id >= RWKV_T_LN1_W && id <= RWKV_T_FFN_X_K) || (id >= RWKV_T_W1 && id <= RWKV_T_V2),
               "set_tensor: unknown tensor id %d", id);
  m->layers[layer].t[id] = p;
  // rank-in matrices [R, C] also get a copy in the MFMA-native order for calls with many rows
  const int w1_ids[4] = {RWKV_T_W1, RWKV_T_A1, RWKV_T_G1, RWKV_T_V1};
  const int ranks[4] = {m->Rw, m->Ra, m->Rg, m->Rv};
  for (int i = 0; i < 4; ++i) {
    if (id != w1_ids[i]) continue;
    void*& slot = m->layers[layer].lora_in_packed[i];
    if (slot) {
      RWKV_HIP_TRY(hipDeviceSynchronize());
      RWKV_HIP_TRY(hipFree(slot));
      slot = nullptr;
    }
    if (linear_packed_supported(RWKV_FMT_F16, kPackedMinRows, ranks[i], m->C)) {
      RWKV_HIP_TRY(hipMalloc(&slot, static_cast<size_t>(ranks[i]) * m->C * 2));
      const int rc = pack_weights_launch(nullptr, RWKV_FMT_F16, ranks[i], m->C, data, slot);
      if (rc != RWKV_OK) return rc;
      RWKV_HIP_TRY(hipStreamSynchronize(nullptr));
    }
  }
  // rank-out matrices [C, R]: a copy in the order the many-row rank-out kernel reads them
  const int w2_ids[4] = {RWKV_T_W2, RWKV_T_A2, RWKV_T_G2, RWKV_T_V2};
  for (int i = 0; i < 4; ++i) {
    if (id != w2_ids[i]) continue;
    half_t*& slot = m->layers[layer].lora_out_packed[i];
    if (slot) {
      RWKV_HIP_TRY(hipDeviceSynchronize());
      RWKV_HIP_TRY(hipFree(slot));
      slot = nullptr;
    }
    if (ranks[i] > 0 && ranks[i] % 8 == 0) {
      RWKV_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&slot), lora_pack_w2_halfs(m->C, ranks[i]) * sizeof(half_t)));
      const int rc = lora_pack_w2_launch(nullptr, m->C, ranks[i], p, slot);
      if (rc != RWKV_OK) return rc;
      RWKV_HIP_TRY(hipStreamSynchronize(nullptr));
    }
  }
  return RWKV_OK;
}

int rwkv_hip_model_set_matrix(rwkv_hip_model* m, int layer, int id, int fmt, const void* data, const void* scale,
                              const void* zp) {
  RWKV_REQUIRE(m && data, "set_matrix: NULL argument");
  RWKV_REQUIRE(fmt == RWKV_FMT_F16 || fmt == RWKV_FMT_W8 || fmt == RWKV_FMT_W4, "set_matrix: bad format %d", fmt);
  RWKV_REQUIRE(fmt == RWKV_FMT_F16 || scale, "set_matrix: quantised matrix needs a scale tensor");
  RWKV_REQUIRE(fmt != RWKV_FMT_W4 || zp, "set_matrix: W4 matrix needs a zero-point tensor");
  Matrix mat;
  mat.fmt = fmt; mat.data = data; mat.scale = static_cast<const half_t*>(scale); mat.zp = static_cast<const uint8_t*>(zp);
  if (id != RWKV_M_HEAD) {
    RWKV_REQUIRE(layer >= 0 && layer < m->L, "set_matrix: layer %d out of range", layer);
    RWKV_REQUIRE(id >= 0 && id < 6, "set_matrix: unknown matrix id %d", id);
  }
  const int N = id == RWKV_M_HEAD ? m->V : (id == RWKV_M_FFN_KEY ? m->F : m->C);
  const int K = id == RWKV_M_FFN_VALUE ? m->F : m->C;
  if (fmt == RWKV_FMT_W4) {
    RWKV_REQUIRE(K % 128 == 0, "set_matrix: W4 needs the input width (%d) to be a multiple of 128", K);
  }
  Matrix& slot = id == RWKV_M_HEAD ? m->head : m->layers[layer].m[id];
  if (slot.packed || slot.sparse_t) {
    RWKV_HIP_TRY(hipDeviceSynchronize());
    if (slot.packed) RWKV_HIP_TRY(hipFree(slot.packed));
    if (slot.sparse_t) RWKV_HIP_TRY(hipFree(slot.sparse_t));
    slot.packed = nullptr;
    slot.sparse_t = nullptr;
  }
  if (linear_packed_supported(fmt, kPackedMinRows, N, K)) {
    // second copy of the codes in the order the MFMA path streams (batched decode and prefill)
    const size_t bytes = fmt == RWKV_FMT_F16 ? static_cast<size_t>(N) * K * 2
                                             : (fmt == RWKV_FMT_W8 ? static_cast<size_t>(N) * K : static_cast<size_t>(N) * K / 2);
    RWKV_HIP_TRY(hipMalloc(&mat.packed, bytes));
    const int rc = pack_weights_launch(nullptr, fmt, N, K, data, mat.packed);
    if (rc != RWKV_OK) {
      (void)hipFree(mat.packed);
      return rc;
    }
    RWKV_HIP_TRY(hipStreamSynchronize(nullptr));
  }
  if (id == RWKV_M_FFN_VALUE && ffn_sparse_supported(fmt, N, K)) {
    // third copy: transposed, for decode steps of one sequence
    RWKV_HIP_TRY(hipMalloc(&mat.sparse_t, ffn_sparse_packed_bytes(fmt, N, K)));
    const int rc = fmt == RWKV_FMT_W4 ? ffn_sparse_pack_w4_launch(nullptr, N, K, data, mat.scale, mat.zp, mat.sparse_t)
                                      : ffn_sparse_pack_launch(nullptr, fmt, N, K, data, mat.sparse_t);
    if (rc != RWKV_OK) {
      (void)hipFree(mat.sparse_t);
      if (mat.packed) (void)hipFree(mat.packed);
      return rc;
    }
    RWKV_HIP_TRY(hipStreamSynchronize(nullptr));
  }
  slot = mat;
  return RWKV_OK;
}

int rwkv_hip_model_weight_bytes(const rwkv_hip_model* m, uint64_t* bytes) {
  RWKV_REQUIRE(m && bytes, "weight_bytes: NULL argument");
  auto mat_bytes = [](const Matrix& mat, uint64_t N, uint64_t K) -> uint64_t {
    switch (mat.fmt) {
      case RWKV_FMT_W8: return N * K + N * 2;
      case RWKV_FMT_W4: return N * K / 2 + N * (K / 128) * 3;
      default: return N * K * 2;
    }
  };
  const uint64_t C = m->C, F = m->F, V = m->V;
  uint64_t total = mat_bytes(m->head, V, C) + 2 * C * 2;  // head + ln_out
  for (int l = 0; l < m->L; ++l) {
    const Layer& w = m->layers[l];
    total += mat_bytes(w.m[RWKV_M_ATT_R], C, C) + mat_bytes(w.m[RWKV_M_ATT_K], C, C) + mat_bytes(w.m[RWKV_M_ATT_V], C, C) +
             mat_bytes(w.m[RWKV_M_ATT_O], C, C) + mat_bytes(w.m[RWKV_M_FFN_KEY], F, C) + mat_bytes(w.m[RWKV_M_FFN_VALUE], C, F);
    total += 19 * C * 2;  // per-layer vectors
    const uint64_t ranks = static_cast<uint64_t>(m->Rw) + m->Ra + m->Rg + (l > 0 ? m->Rv : 0);
    total += 2 * ranks * C * 2;  // LoRA pairs, fp16
  }
  *bytes = total;
  return RWKV_OK;
}

int rwkv_hip_session_create(rwkv_hip_session** out, const rwkv_hip_model* m) {
  RWKV_REQUIRE(out && m, "session_create: NULL argument");
  *out = nullptr;
  rwkv_hip_session* s = new (std::nothrow) rwkv_hip_session();
  if (!s) {
    set_error("session: out of host memory");
    return RWKV_E_NOMEM;
  }
  s->model = m;

  const hipError_t err = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
  if (err != hipSuccess) {
    set_error("hipStreamCreateWithFlags failed: %s", hipGetErrorString(err));
    delete s;
    return RWKV_E_RUNTIME;
  }
  *out = s;
  return RWKV_OK;
}

int rwkv_hip_session_destroy(rwkv_hip_session* s) {
  if (!s) return RWKV_OK;
  (void)hipStreamSynchronize(s->stream);
  for (auto& g : s->graphs) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (g.graph) (void)hipGraphDestroy(g.graph);
  }
  if (s->arena.base) (void)hipFree(s->arena.base);
  if (s->gemm_ws) (void)hipFree(s->gemm_ws);
  if (s->sparse_ws) (void)hipFree(s->sparse_ws);
  if (s->tokens_dev) (void)hipFree(s->tokens_dev);
  if (s->tokens_pinned) (void)hipHostFree(s->tokens_pinned);
  if (s->argmax_dev) (void)hipFree(s->argmax_dev);
  if (s->history_dev) (void)hipFree(s->history_dev);
  (void)hipStreamDestroy(s->stream);
  delete s;
  return RWKV_OK;
}

int rwkv_hip_session_stream(rwkv_hip_session* s, rwkv_stream_t* stream) {
  RWKV_REQUIRE(s && stream, "session_stream: NULL argument");
  *stream = s->stream;
  return RWKV_OK;
}

int rwkv_hip_session_set_graph(rwkv_hip_session* s, int use_graph) {
  RWKV_REQUIRE(s, "session is NULL");
  s->use_graph = use_graph != 0;
  return RWKV_OK;
}

int rwkv_hip_session_set_profile(rwkv_hip_session* s, int on) {
  RWKV_REQUIRE(s, "session is NULL");
  RWKV_REQUIRE(on >= 0 && on <= 2, "set_profile: mode must be 0, 1 or 2");
  s->profile = on;
  return RWKV_OK;
}

static int drop_graphs(rwkv_hip_session* s) {
  RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  for (auto& g : s->graphs) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (g.graph) (void)hipGraphDestroy(g.graph);
  }
  s->graphs.clear();
  return RWKV_OK;
}

int rwkv_hip_graph_capture_count(int64_t* count) {
  RWKV_REQUIRE(count != nullptr, "count is NULL");
  *count = g_graph_captures.load(std::memory_order_relaxed);
  return RWKV_OK;
}

int rwkv_hip_session_set_fused_ln(rwkv_hip_session* s, int on) {
  RWKV_REQUIRE(s, "session is NULL");
  const int want = on < 0 ? -1 : (on != 0);
  if (s->fused_ln != want) {
    TRY(drop_graphs(s));  // captured decode graphs hold the other kernels
    s->fused_ln = want;
  }
  return RWKV_OK;
}

int rwkv_hip_session_set_tmix_rows(rwkv_hip_session* s, int rows) {
  RWKV_REQUIRE(s, "session is NULL");
  RWKV_REQUIRE(rows < 0 || rows == 0 || rows == 1 || rows == 2 || rows == 4, "rows per block: 1, 2 or 4; 0 or < 0");
  const int want = rows < 0 ? -1 : rows;
  if (s->tmix_rows != want) {
    TRY(drop_graphs(s));  // captured decode graphs hold the other kernels
    s->tmix_rows = want;
  }
  return RWKV_OK;
}

int rwkv_hip_session_set_wkv_fp16(rwkv_hip_session* s, int on) {
  RWKV_REQUIRE(s, "session is NULL");
  const bool want = on != 0;
  if (s->wkv_fp16 != want) {
    TRY(drop_graphs(s));  // captured decode graphs hold the other recurrence kernel
    s->wkv_fp16 = want;
  }
  return RWKV_OK;
}

int rwkv_hip_session_set_sparse_ffn(rwkv_hip_session* s, int max_rows) {
  RWKV_REQUIRE(s, "session is NULL");
  RWKV_REQUIRE(max_rows >= 0 && max_rows <= kSparseMaxRows, "set_sparse_ffn: max_rows %d out of range (0..%d)", max_rows,
               kSparseMaxRows);
  if (s->sparse_ffn_rows != max_rows) {
    TRY(drop_graphs(s));  // captured decode graphs hold the other kernel
    s->sparse_ffn_rows = max_rows;
  }
  return RWKV_OK;
}

int rwkv_hip_session_read_profile(rwkv_hip_session* s, int64_t* launches, double* total_ms) {
  RWKV_REQUIRE(s && launches && total_ms, "read_profile: NULL argument");
  RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  double ms = 0.0;
  for (auto& pr : s->prof_events) {
    float t = 0.0f;
    RWKV_HIP_TRY(hipEventElapsedTime(&t, pr.first, pr.second));
    ms += t;
    (void)hipEventDestroy(pr.first);
    (void)hipEventDestroy(pr.second);
  }
  *launches = s->prof_launches;
  *total_ms = ms;
  s->prof_events.clear();
  s->prof_launches = 0;
  return RWKV_OK;
}

int rwkv_hip_session_debug_buffer(rwkv_hip_session* s, int id, void** ptr) {
  RWKV_REQUIRE(s && ptr, "debug_buffer: NULL argument");
  const Buffers& b = s->buf;
  void* table[] = {b.x,  b.xx,  b.xr,  b.xw, b.xk, b.xv,  b.xa,  b.xg, b.r,   b.k,     b.v,  b.v_first,
                   b.w12, b.a12, b.g,  b.hw, b.ha, b.hg,  b.hv,  b.k2, b.nkk, b.kka,   b.y,  b.y2,
                   b.att, b.x1,  b.ln2, b.mixed, b.act, b.cm, b.r32, b.d32, b.k32, b.a32, b.b32};
  RWKV_REQUIRE(id >= 0 && id < static_cast<int>(sizeof(table) / sizeof(table[0])), "debug_buffer: unknown id %d", id);
  *ptr = table[id];
  return RWKV_OK;
}

int rwkv_hip_session_set_trace(rwkv_hip_session* s, void* trace) {
  RWKV_REQUIRE(s, "session is NULL");
  s->trace = static_cast<half_t*>(trace);
  return RWKV_OK;
}

int rwkv_hip_forward(rwkv_hip_session* s, const int64_t* tokens_host, int B, int T, void* shift, void* wkv,
                     void* elapsed, void* logits, int sync) {
  TRY(check_forward_args(s, B, T, shift, wkv, elapsed, logits));
  RWKV_REQUIRE(tokens_host != nullptr, "forward: tokens is NULL");
  const int rows = B * T;
  for (int i = 0; i < rows; ++i) {
    RWKV_REQUIRE(tokens_host[i] >= 0 && tokens_host[i] < s->model->V, "token id out of range");  // :1107-1110
  }
  TRY(ensure_arena(s, B, T));
  // the pinned staging buffer may still be in flight from the previous call
  RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  std::copy(tokens_host, tokens_host + rows, s->tokens_pinned);
  RWKV_HIP_TRY(hipMemcpyAsync(s->tokens_dev, s->tokens_pinned, sizeof(int64_t) * rows, hipMemcpyHostToDevice, s->stream));
  if (T == 1) {
    TRY(run_step(s, B, static_cast<half_t*>(shift), wkv, static_cast<int*>(elapsed), static_cast<float*>(logits)));
  } else {
    TRY(enqueue_forward(s, B, T, static_cast<half_t*>(shift), wkv, static_cast<int*>(elapsed), static_cast<float*>(logits)));
  }
  if (sync) RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  return RWKV_OK;
}

int rwkv_hip_decode_greedy(rwkv_hip_session* s, const int64_t* first_tokens_host, int B, int steps, void* shift,
                           void* wkv, void* elapsed, void* logits, int32_t* out_tokens_host) {
  TRY(check_forward_args(s, B, 1, shift, wkv, elapsed, logits));
  RWKV_REQUIRE(first_tokens_host && out_tokens_host && steps > 0, "decode_greedy: bad arguments");
  for (int i = 0; i < B; ++i)
    RWKV_REQUIRE(first_tokens_host[i] >= 0 && first_tokens_host[i] < s->model->V, "token id out of range");
  TRY(ensure_arena(s, B, 1));
  RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  if (B > s->argmax_cap) {
    if (s->argmax_dev) RWKV_HIP_TRY(hipFree(s->argmax_dev));
    s->argmax_dev = nullptr;
    s->argmax_cap = 0;
    RWKV_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&s->argmax_dev), sizeof(int) * B));
    s->argmax_cap = B;
  }
  const size_t hist = static_cast<size_t>(steps) * B;
  if (hist > s->history_cap) {
    if (s->history_dev) RWKV_HIP_TRY(hipFree(s->history_dev));
    s->history_dev = nullptr;
    s->history_cap = 0;
    RWKV_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&s->history_dev), sizeof(int) * hist));
    s->history_cap = hist;
  }
  std::copy(first_tokens_host, first_tokens_host + B, s->tokens_pinned);
  RWKV_HIP_TRY(hipMemcpyAsync(s->tokens_dev, s->tokens_pinned, sizeof(int64_t) * B, hipMemcpyHostToDevice, s->stream));
  for (int i = 0; i < steps; ++i) {
    TRY(run_step(s, B, static_cast<half_t*>(shift), wkv, static_cast<int*>(elapsed), static_cast<float*>(logits)));
    // the picked ids are the next step's input tokens and step i of the list that goes back to the host
    TRY(argmax_launch(s->stream, B, s->model->V, static_cast<float*>(logits), s->argmax_dev, s->tokens_dev,
                      s->history_dev + static_cast<size_t>(i) * B));
  }
  RWKV_HIP_TRY(hipMemcpyAsync(out_tokens_host, s->history_dev, sizeof(int) * hist, hipMemcpyDeviceToHost, s->stream));
  RWKV_HIP_TRY(hipStreamSynchronize(s->stream));
  return RWKV_OK;
}

}  // extern "C"
