// WKV7 time-mix recurrence for gfx950, fp32 state.
//
// Reference semantics: cuda/rwkv7_wkv_fp32_v2.cu:100-126 (per token, thread i owns state row i):
//   sa = sum_j S[i][j]*a[j];  S[i][j] = S[i][j]*d[j] + sa*b[j] + k[j]*v[i];  y[i] = sum_j S[i][j]*r[j]
// with the decay map d = exp(-e^-1/2 * sigmoid(w)) of :13-14,26-28.
//
// Sequence kernel (any T): four to sixteen wavefronts per (batch, head), each lane keeps a few rows x 4 columns of
// the 64 x 64 state in registers for the whole call.  The per-column operands r,d,k,a,b of a token are staged in
// LDS as fp32 and each lane reads only the four columns it owns; the two row sums of a step (sa and y) are
// reduced over the 16 lanes that share a row with DPP adds.  The staging converts what the caller has (fp16 or
// fp32 tensors, raw decay logits or decays, or the model's own fp16 rows) on the way into LDS.
#include <type_traits>
#include "ops.h"

namespace rwkv {

constexpr float kWScaleLog2e = -0.8750387749145276f;  // -e^-1/2 * log2(e), rwkv7_wkv_fp32_v2.cu:13
constexpr float kNLog2e = -1.4426950408889634f;       // rwkv7_wkv_fp32_v2.cu:14

__device__ __forceinline__ float decay_from_logit(float w) {
  return exp2f(kWScaleLog2e / (1.0f + exp2f(kNLog2e * w)));
}

// ---- sequence kernel -------------------------------------------------------------------------
// grid = B*H, block = 1024/RPL threads: 16/RPL wavefronts per head, RPL = 4, 2 or 1 state rows per lane.  Lane
// (g, c) = (lane / 16, lane % 16) of wavefront q owns rows 4*RPL*q + RPL*g .. +RPL-1 and columns 4c .. 4c+3, so
// the 16 lanes of one DPP row hold complete state rows and the wavefronts never exchange data.  r,d,k,a,b are
// fp32 with `op_bs` elements between batch rows; v,y are IO with `io_bs` elements between batch rows.  The
// block stages the operands kSeqChunk tokens at a time with coalesced 16-byte loads, double-buffered (the
// loads of chunk c+1 are in flight while chunk c computes); a step costs each lane six LDS reads (its four
// columns of the five operands and its v values) against 28*RPL VALU operations.  y goes back through LDS so
// that the global stores are coalesced.  The arithmetic of a state element does not depend on RPL or on the
// chunking: every variant and every split of T over several calls gives bitwise the same result.  Smaller RPL
// means less serial work per token and wavefront and is used while the grid is small enough to leave SIMDs
// idle (RPL = 1 up to 64 heads, 2 up to 128); RPL = 4 reads each operand least often.
constexpr int kSeqChunk = 8;

// Where the five operand vectors of a token come from (SRC):
//   kSrcFp32  - fp32 tensors r, d, k, a, b (decay applied), `op_bs` elements between batch rows, staged with 16-byte
//               loads: what kk_a_gate_kernel writes for the model's stand-alone path;
//   kSrcRaw   - the caller's r, w, k, a, b in the io type, converted (and the decay derived from w, by w_mode)
//               while staging, one wavefront per token, lane = channel: the C-ABI operator, which so reads every
//               operand once instead of through an fp32 copy (14 instead of 56 bytes per token and channel);
//   kSrcFused - the model's fused pass, below.
constexpr int kSrcFp32 = 0;
constexpr int kSrcFused = 1;
constexpr int kSrcRaw = 2;
struct RawOperands {
  const void *r, *w, *k, *a, *b;
  int w_mode;
};

// FUSED (the model's row-tiled time-mix path, fp16 io): the operands are not read as fp32 tensors but derived
// while staging from the fp16 rows r, k, a12, w12 - the arithmetic of kk_a_gate_kernel, one wavefront per token,
// lane = channel - and y is not stored but taken through the per-head GroupNorm, the (r.k.r_k) v bonus and the
// gate - the arithmetic of lnx_rkvres_xg_kernel on the fp16-rounded y - so that three launches and the fp32
// operand tensors between them become one launch.  Bitwise the same results as the three kernels.
//
// PARTS > 1: the rows of a head's state are independent of each other (row i needs only its own sum over the
// columns, v_i and the per-column operands), so a head is cut into PARTS row ranges that run as separate blocks on
// separate CUs - with few heads in flight the step is bound by one CU's VALU rate, not by memory.  Not with FUSED
// (the GroupNorm needs the whole head's y).  Same lanes, same rows, same arithmetic: bitwise the same results.
//
// STRAIGHT = false leaves out the unrolled eight-step body: single-token calls move a head's state once and are
// bound by that traffic, so they want the registers for more blocks per CU instead (148 -> under 100 VGPRs).
template <typename IO, int RPL, int PARTS, int SRC, bool STRAIGHT = true>
__global__ __launch_bounds__(1024 / RPL / PARTS) void wkv7_seq_kernel(int T, int C, int H, float* __restrict__ state,
                                                              const float* __restrict__ r, const float* __restrict__ d,
                                                              const float* __restrict__ k, const float* __restrict__ a,
                                                              const float* __restrict__ b, int64_t op_bs,
                                                              const IO* __restrict__ v, IO* __restrict__ y,
                                                              int64_t io_bs, TmixSeqArgs fa, RawOperands ro) {
  constexpr bool FUSED = SRC == kSrcFused;
  constexpr bool RAW = SRC == kSrcRaw;
  static_assert(PARTS == 1 || !FUSED, "the fused pass needs whole heads");
  constexpr int NT = 1024 / RPL / PARTS;
  constexpr int kOpVecs = 5 * kSeqChunk * (kHead / 4);         // float4 of operands per chunk
  constexpr int kOpSlots = (kOpVecs + NT - 1) / NT;
  constexpr int kVSlots = (kSeqChunk * kHead + NT - 1) / NT;
  typedef float rows_t __attribute__((ext_vector_type(RPL)));
  __shared__ __align__(16) float ops[2][kSeqChunk][5][kHead];  // [buffer][token][a,b,d,k,r][column]
  __shared__ __align__(16) float vs[2][kSeqChunk][kHead];      // [buffer][token][row]
  __shared__ __align__(16) float ys[2][kSeqChunk][kHead];
  // Where to the 15 idle lanes of a row store in step_out.  The single-token variant keeps to 32 KB of LDS instead
  // (five blocks per CU) and stores under a branch.
  constexpr bool kSpare = STRAIGHT;
  __shared__ __align__(16) float spare[kSpare ? NT * RPL : 4];
  __shared__ __align__(16) float gs[FUSED ? 2 : 1][FUSED ? kSeqChunk : 1][kHead];  // FUSED: the gate rows

  const int bh = blockIdx.x / PARTS;
  const int part = blockIdx.x % PARTS;
  const int bi = bh / H;
  const int h = bh - bi * H;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int row_lo = part * (kHead / PARTS);                         // this block's rows
  const int i0 = row_lo + 4 * RPL * (tid >> 6) + RPL * (lane >> 4);  // first of this lane's rows
  const int j0 = 4 * (lane & 15);                           // first of its 4 columns
  float* sblk = state + (static_cast<int64_t>(bh) * kHead + i0) * kHead + j0;

  float4_t S[RPL];
#pragma unroll
  for (int i = 0; i < RPL; ++i) S[i] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(sblk + i * kHead));

  const int64_t base = static_cast<int64_t>(bi) * op_bs + h * kHead;
  const int64_t iob = static_cast<int64_t>(bi) * io_bs + h * kHead;
  // staging slot i of thread t: float4 number t + i*NT of the chunk = (operand, token, 4 columns)
  const float* st_src[kOpSlots];
  int st_tok[kOpSlots];
  int st_dst[kOpSlots];  // offset inside ops[buf], -1: slot unused
#pragma unroll
  for (int i = 0; i < kOpSlots; ++i) {
    const int idx = tid + i * NT;
    const int o = idx / (kSeqChunk * 16);
    const int tok = (idx >> 4) % kSeqChunk;
    const int col = (idx & 15) * 4;
    const float* src = o == 0 ? a : (o == 1 ? b : (o == 2 ? d : (o == 3 ? k : r)));
    st_src[i] = src + base + col;
    st_tok[i] = tok;
    st_dst[i] = idx < kOpVecs ? (tok * 5 + o) * kHead + col : -1;
  }

  // Two sets of staging registers: a chunk is requested two chunks before it is needed - eight steps are shorter
  // than a trip to memory.
  float4_t stage[2][kOpSlots];
  float v_stage[2][kVSlots];
  // FUSED: raw fp16 values of this thread's (token, channel) slots: r, k, a12, w12, g; and its channel's constants
  half_t raw[2][kVSlots][5];
  // RAW: the caller's r, w, k, a, b values of the slots, still in the io type
  IO rio[2][RAW ? kVSlots : 1][5];
  const IO* ro_r = static_cast<const IO*>(ro.r);
  const IO* ro_w = static_cast<const IO*>(ro.w);
  const IO* ro_k = static_cast<const IO*>(ro.k);
  const IO* ro_a = static_cast<const IO*>(ro.a);
  const IO* ro_b = static_cast<const IO*>(ro.b);
  float c_kk = 0.0f, c_a0 = 0.0f, c_ka = 0.0f, c_w0 = 0.0f, c_rk = 0.0f, c_lnw = 0.0f, c_lnb = 0.0f;
  if constexpr (FUSED) {
    const int c = h * kHead + lane;
    c_kk = h2f(fa.k_k[c]); c_a0 = h2f(fa.a0[c]); c_ka = h2f(fa.k_a[c]); c_w0 = h2f(fa.w0[c]);
    c_rk = h2f(fa.r_k[c]); c_lnw = h2f(fa.lnx_w[c]); c_lnb = h2f(fa.lnx_b[c]);
  }

  // Every load is issued unconditionally (tokens past the end repeat the last one; their steps never run): a load
  // under a branch makes the compiler's s_waitcnt accounting wait for everything in flight, the younger set too.
  auto request = [&](int t0, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    if constexpr (SRC == kSrcFp32) {
#pragma unroll
      for (int i = 0; i < kOpSlots; ++i) {
        stage[set][i] = *reinterpret_cast<const float4_t*>(st_src[i] + static_cast<int64_t>(min(t0 + st_tok[i], T - 1)) * C);
      }
    }
#pragma unroll
    for (int i = 0; i < kVSlots; ++i) {
      const int tok = min((tid + i * NT) >> 6, kSeqChunk - 1);
      const int64_t at = iob + static_cast<int64_t>(min(t0 + tok, T - 1)) * C + lane;
      v_stage[set][i] = static_cast<float>(v[at]);
      if constexpr (FUSED) {
        raw[set][i][0] = fa.r[at]; raw[set][i][1] = fa.k[at]; raw[set][i][2] = fa.a12[at]; raw[set][i][3] = fa.w12[at];
        raw[set][i][4] = fa.g[at];
      }
      if constexpr (RAW) {
        rio[set][i][0] = ro_a[at]; rio[set][i][1] = ro_b[at]; rio[set][i][2] = ro_w[at]; rio[set][i][3] = ro_k[at];
        rio[set][i][4] = ro_r[at];
      }
    }
  };
  auto commit = [&](int buf, auto set_c) {
    constexpr int set = decltype(set_c)::value;
    if constexpr (SRC == kSrcFp32) {
#pragma unroll
      for (int i = 0; i < kOpSlots; ++i)
        if (st_dst[i] >= 0) *reinterpret_cast<float4_t*>(&ops[buf][0][0][0] + st_dst[i]) = stage[set][i];
    }
#pragma unroll
    for (int i = 0; i < kVSlots; ++i) {
      const int tok = (tid + i * NT) >> 6;  // wave-uniform: one wavefront per token, lane = channel
      if (tok < kSeqChunk) {
        vs[buf][tok][lane] = v_stage[set][i];
        if constexpr (FUSED) {
          // kk normalise, a-gate, new k, decay: the statements of kk_a_gate_kernel
          const float kv = h2f(raw[set][i][1]);
          const float u = kv * c_kk;
          const float total = wave_sum(u * u);
          const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
          const float kk = u * inv;
          const float av = sigmoid_f(c_a0 + h2f(raw[set][i][2]));
          const half_t nk = f2h(kv * fmaf(av, c_ka, 1.0f - c_ka));
          const half_t nkk = f2h(-kk);
          const half_t kka = f2h(kk * av);
          const float wraw = round_h(h2f(raw[set][i][3]) + c_w0);
          ops[buf][tok][0][lane] = h2f(nkk);
          ops[buf][tok][1][lane] = h2f(kka);
          ops[buf][tok][2][lane] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
          ops[buf][tok][3][lane] = h2f(nk);
          ops[buf][tok][4][lane] = h2f(raw[set][i][0]);
          gs[buf][tok][lane] = h2f(raw[set][i][4]);
        }
        if constexpr (RAW) {
          const float wv = static_cast<float>(rio[set][i][2]);
          ops[buf][tok][0][lane] = static_cast<float>(rio[set][i][0]);
          ops[buf][tok][1][lane] = static_cast<float>(rio[set][i][1]);
          ops[buf][tok][2][lane] = (ro.w_mode == RWKV_W_RAW_LOGIT) ? decay_from_logit(wv) : wv;
          ops[buf][tok][3][lane] = static_cast<float>(rio[set][i][3]);
          ops[buf][tok][4][lane] = static_cast<float>(rio[set][i][4]);
        }
      }
    }
  };

  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  request(0, Set0{});
  if (T > kSeqChunk) request(kSeqChunk, Set1{});
  commit(0, Set0{});
  __syncthreads();
  // The y rows of a finished chunk (tokens t0 .. t0+n-1, LDS buffer buf) go to memory: one wavefront per token,
  // lane = channel.  It runs in the middle of the next chunk, where its LDS and memory latencies hide behind the
  // steps; ys[buf] is next written a barrier later.  FUSED also reads the chunk's operand, v and gate rows: each
  // thread reads exactly the (token, channel) slots that it overwrites itself in the commit that follows.
  auto write_out = [&](int t0, int n, int buf) {
#pragma unroll
    for (int i = 0; i < kVSlots; ++i) {
      const int tt = (tid + i * NT) >> 6;
      if (tt < n) {
        if constexpr (FUSED) {
          // GroupNorm over the head, (r.k.r_k) v bonus, gate: the statements of lnx_rkvres_xg_kernel on the
          // fp16-rounded y
          const float yv = round_h(ys[buf][tt][lane]);
          const float mean = wave_sum(yv) * (1.0f / 64.0f);
          const float dd = yv - mean;
          const float var = wave_sum(dd * dd) * (1.0f / 64.0f);
          const float rstd = rsqrtf(var + kLnxEps);
          const float rkv = wave_sum(ops[buf][tt][4][lane] * ops[buf][tt][3][lane] * c_rk);
          const float o = (dd * rstd * c_lnw + c_lnb + rkv * vs[buf][tt][lane]) * gs[buf][tt][lane];
          y[iob + static_cast<int64_t>(t0 + tt) * C + lane] = static_cast<IO>(o);
        } else if (PARTS == 1 || (lane >= row_lo && lane < row_lo + kHead / PARTS)) {
          y[iob + static_cast<int64_t>(t0 + tt) * C + lane] = static_cast<IO>(ys[buf][tt][lane]);
        }
      }
    }
  };
  // chunk c: LDS buffer c&1, staging set c&1 - both static inside the two-chunk body
  auto run_chunk = [&](int t0, auto set_c) {
    constexpr int buf = decltype(set_c)::value;
    using Other = std::integral_constant<int, 1 - buf>;
    const bool more = t0 + kSeqChunk < T;
    request(t0 + 2 * kSeqChunk, set_c);  // this chunk's set was committed a chunk ago
    const int n = min(kSeqChunk, T - t0);
    struct StepOps {
      float4_t av, bv, dv, kv, rv;
      rows_t vv;
    };
    auto load_step = [&](int tt, StepOps& q) {
      q.av = *reinterpret_cast<const float4_t*>(&ops[buf][tt][0][j0]);
      q.bv = *reinterpret_cast<const float4_t*>(&ops[buf][tt][1][j0]);
      q.dv = *reinterpret_cast<const float4_t*>(&ops[buf][tt][2][j0]);
      q.kv = *reinterpret_cast<const float4_t*>(&ops[buf][tt][3][j0]);
      q.rv = *reinterpret_cast<const float4_t*>(&ops[buf][tt][4][j0]);
      q.vv = *reinterpret_cast<const rows_t*>(&vs[buf][tt][i0]);
    };
    // A step in two halves.  step_state carries the recurrence: row sums of S a, then the update - the only chain
    // from one token to the next.  step_out reads the new state: y = S r.
    auto step_state = [&](const StepOps& q) {
      const float4_t av = q.av, bv = q.bv, dv = q.dv, kv = q.kv;
      float sa[RPL];
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        float p = S[i].x * av.x;
        p = fmaf(S[i].y, av.y, p);
        p = fmaf(S[i].z, av.z, p);
        p = fmaf(S[i].w, av.w, p);
        sa[i] = p;
      }
#pragma unroll
      for (int i = 0; i < RPL; ++i) sa[i] = row16_sum(sa[i]);
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        const float vi = q.vv[i];
        S[i].x = fmaf(S[i].x, dv.x, fmaf(sa[i], bv.x, kv.x * vi));
        S[i].y = fmaf(S[i].y, dv.y, fmaf(sa[i], bv.y, kv.y * vi));
        S[i].z = fmaf(S[i].z, dv.z, fmaf(sa[i], bv.z, kv.z * vi));
        S[i].w = fmaf(S[i].w, dv.w, fmaf(sa[i], bv.w, kv.w * vi));
      }
    };
    auto step_out = [&](int tt, const StepOps& q) {
      const float4_t rv = q.rv;
      rows_t yy;
#pragma unroll
      for (int i = 0; i < RPL; ++i) {
        float p = S[i].x * rv.x;
        p = fmaf(S[i].y, rv.y, p);
        p = fmaf(S[i].z, rv.z, p);
        p = fmaf(S[i].w, rv.w, p);
        yy[i] = p;
      }
#pragma unroll
      for (int i = 0; i < RPL; ++i) yy[i] = row16_sum(yy[i]);
      // the 16 lanes of a row hold the same sums: the first stores them, the others store to a spare area - a
      // store under a branch would end the scheduling region here
      if constexpr (kSpare) {
        float* dst = (lane & 15) == 0 ? &ys[buf][tt][i0] : &spare[tid * RPL];
        *reinterpret_cast<rows_t*>(dst) = yy;
      } else {
        if ((lane & 15) == 0) *reinterpret_cast<rows_t*>(&ys[buf][tt][i0]) = yy;
      }
    };
    if (STRAIGHT && n == kSeqChunk) {
      // Full chunk, straight-line.  The operands of step tt+1 are read from LDS while step tt computes, and the
      // scheduling regions run from the middle of one step to the middle of the next
      // (__builtin_amdgcn_sched_barrier(0) between the halves), so that the compiler fills the latency bubbles
      // of step tt's output sums with the independent recurrence half of step tt+1.
      StepOps q[2];
      load_step(0, q[0]);
#pragma unroll
      for (int tt = 0; tt < kSeqChunk; ++tt) {
        if (tt + 1 < kSeqChunk) load_step(tt + 1, q[(tt + 1) & 1]);
        step_state(q[tt & 1]);
        __builtin_amdgcn_sched_barrier(0);
        step_out(tt, q[tt & 1]);
        if (tt == kSeqChunk / 2 - 1) {
          if (t0 > 0) write_out(t0 - kSeqChunk, kSeqChunk, buf ^ 1);
          if (more) commit(buf ^ 1, Other{});
        }
      }
    } else {
      // the last, partial chunk (and single-token calls): same step arithmetic, rolled loop
#pragma unroll 1
      for (int tt = 0; tt < n; ++tt) {
        StepOps q;
        load_step(tt, q);
        step_state(q);
        step_out(tt, q);
      }
      if (t0 > 0) write_out(t0 - kSeqChunk, kSeqChunk, buf ^ 1);
      if (more) commit(buf ^ 1, Other{});  // (only without the straight-line body: a partial chunk is the last)
    }
    __syncthreads();
  };
  for (int t0 = 0; t0 < T; t0 += 2 * kSeqChunk) {
    run_chunk(t0, Set0{});
    if (t0 + kSeqChunk < T) run_chunk(t0 + kSeqChunk, Set1{});
  }
  const int t_last = (T - 1) / kSeqChunk * kSeqChunk;
  write_out(t_last, T - t_last, (t_last / kSeqChunk) & 1);

#pragma unroll
  for (int i = 0; i < RPL; ++i) __builtin_nontemporal_store(S[i], reinterpret_cast<float4_t*>(sblk + i * kHead));
}

// Heads in flight up to which a head is cut into four (two) row ranges of four wavefronts each, one block per
// range; above, one block of four wavefronts per head fills the chip.  Single-token calls move a head's state once
// and are bound by that traffic: whole heads.
constexpr int kSeqSmallGrid = 128;
constexpr int kSeqTinyGrid = 64;

bool tmix_seq_whole_heads(int B, int T, int H) { return !(B * H <= kSeqSmallGrid && T > 1); }

template <typename IO, int SRC>
static void launch_seq(hipStream_t st, int B, int T, int C, int H, float* state, const float* r, const float* d,
                       const float* k, const float* a, const float* b, int64_t op_bs, const IO* v, IO* y, int64_t io_bs,
                       const TmixSeqArgs& fa, const RawOperands& ro) {
  if constexpr (SRC != kSrcFused) {
    if (B * H <= kSeqTinyGrid && T > 1) {
      hipLaunchKernelGGL((wkv7_seq_kernel<IO, 1, 4, SRC>), dim3(B * H * 4), dim3(256), 0, st, T, C, H, state, r, d, k, a, b,
                         op_bs, v, y, io_bs, fa, ro);
      return;
    }
    if (B * H <= kSeqSmallGrid && T > 1) {
      hipLaunchKernelGGL((wkv7_seq_kernel<IO, 2, 2, SRC>), dim3(B * H * 2), dim3(256), 0, st, T, C, H, state, r, d, k, a, b,
                         op_bs, v, y, io_bs, fa, ro);
      return;
    }
  }
  if (T == 1) {
    hipLaunchKernelGGL((wkv7_seq_kernel<IO, 4, 1, SRC, false>), dim3(B * H), dim3(256), 0, st, T, C, H, state, r, d, k, a, b,
                       op_bs, v, y, io_bs, fa, ro);
  } else {
    hipLaunchKernelGGL((wkv7_seq_kernel<IO, 4, 1, SRC>), dim3(B * H), dim3(256), 0, st, T, C, H, state, r, d, k, a, b, op_bs,
                       v, y, io_bs, fa, ro);
  }
}

// The C-ABI operator: operands in the io type, read once by the sequence kernel itself.
template <typename IO>
static int launch_wkv7(hipStream_t st, int B, int T, int C, int H, int w_mode, float* state, const IO* r,
                       const IO* w, const IO* k, const IO* v, const IO* a, const IO* b, IO* y) {
  const int64_t row = static_cast<int64_t>(T) * C;
  const RawOperands ro = {r, w, k, a, b, w_mode};
  launch_seq<IO, kSrcRaw>(st, B, T, C, H, state, nullptr, nullptr, nullptr, nullptr, nullptr, 0, v, y, row, TmixSeqArgs{}, ro);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int wkv7_seq_f16_launch(hipStream_t st, int B, int T, int C, int H, float* state, const float* r, const float* d,
                        const float* k, const float* a, const float* b, int64_t op_bs, const half_t* v, half_t* y,
                        int64_t io_bs) {
  launch_seq<half_t, kSrcFp32>(st, B, T, C, H, state, r, d, k, a, b, op_bs, v, y, io_bs, TmixSeqArgs{}, RawOperands{});
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int tmix_seq_launch(hipStream_t st, int B, int T, int C, int H, float* state, const TmixSeqArgs& fa, const half_t* v,
                    half_t* y2) {
  RWKV_REQUIRE(fa.r && fa.k && fa.a12 && fa.w12 && fa.g && fa.k_k && fa.a0 && fa.k_a && fa.w0 && fa.r_k && fa.lnx_w && fa.lnx_b,
               "tmix_seq: NULL tensor");
  const int64_t row = static_cast<int64_t>(T) * C;
  launch_seq<half_t, kSrcFused>(st, B, T, C, H, state, nullptr, nullptr, nullptr, nullptr, nullptr, 0, v, y2, row, fa,
                                RawOperands{});
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" int rwkv_hip_wkv7(rwkv_stream_t s, int B, int T, int C, int H, int w_mode, int io, void* state,
                             const void* r, const void* w, const void* k, const void* v, const void* a,
                             const void* b, void* y) {
  RWKV_REQUIRE(B > 0 && T > 0 && H > 0, "wkv7: B, T, H must be positive (got %d, %d, %d)", B, T, H);
  RWKV_REQUIRE(C == H * kHead, "wkv7: C (%d) must equal H*64 (%d)", C, H * kHead);
  RWKV_REQUIRE(w_mode == RWKV_W_RAW_LOGIT || w_mode == RWKV_W_DECAY, "wkv7: bad w_mode %d", w_mode);
  RWKV_REQUIRE(state && r && w && k && v && a && b && y, "wkv7: NULL tensor");
  if (io == RWKV_IO_F16) {
    return launch_wkv7<half_t>(as_stream(s), B, T, C, H, w_mode, static_cast<float*>(state),
                               static_cast<const half_t*>(r), static_cast<const half_t*>(w),
                               static_cast<const half_t*>(k), static_cast<const half_t*>(v),
                               static_cast<const half_t*>(a), static_cast<const half_t*>(b),
                               static_cast<half_t*>(y));
  }
  RWKV_REQUIRE(io == RWKV_IO_F32, "wkv7: bad io %d", io);
  return launch_wkv7<float>(as_stream(s), B, T, C, H, w_mode, static_cast<float*>(state),
                            static_cast<const float*>(r), static_cast<const float*>(w),
                            static_cast<const float*>(k), static_cast<const float*>(v),
                            static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(y));
}
