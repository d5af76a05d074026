// WKV7 recurrence with the state kept in fp16: the reference server's default mode (ModelBackend's
// use_wkv32 == false).
//
// Reference: cuda/rwkv7_wkv_fp16_v2.cu - the per-token arithmetic is the same in every kernel of that file
// (:157-193, :342-367, :433-468, :531-556, :632-660): thread i owns state row i as 32 half2 pairs and every operation
// is a packed fp16 fused multiply-add with one rounding (__hfma2),
//   sa2 = chain over pairs j of fma(a[j], S[i][j], sa2);  sa = f16(sa2.x + sa2.y)
//   wd[c] = f16(exp2f(-e^-1/2 log2e / (1 + exp2f(-log2e * w[c]))) - 1 + dither(elapsed[b] + h*64 + c + t))   (:41-52)
//   S[i][j] = fma(S[i][j], wd[j], fma(k[j], v[i], fma(sa, b[j], S[i][j])))
//   y2 = chain over pairs of fma(S'[i][j], r[j], y2);  y[i] = f16(y2.x + y2.y)
// with dither(x) = 2^-41 * float(int32(2654435769 * x)): below the fp16 resolution of d - 1, it makes the rounding of
// the decay unbiased over consecutive tokens and channels.  The order of the two chains is part of the result (fp16
// sums do not associate), so it is kept: the kernel is bit-identical to a scalar restatement of the reference except
// where v_exp_f32 and the host's exp2f differ in the last bit before the decay delta is rounded to fp16.
//
// gfx950 layout: one wavefront per (batch row, head), lane = state row, the row's 64 values in 32 registers as half2
// pairs (v_pk_fma_f16 does both columns of a pair).  The five per-column vectors of a token (a, b, k, decay delta,
// r) are the same for every lane: lane c fetches element c of each for the NEXT token while the current one is
// computed, converts its decay logit, and drops them into LDS, from where every lane reads them back as 16-byte
// broadcasts.  The state is read and written once per call, 16 bytes per lane and instruction.
#include "wkv7_f16state.h"

namespace rwkv {

namespace {

constexpr int kPairs = kPairs16;
constexpr int kAhead = 4;  // tokens whose operands are in flight

struct TokenOps {  // one token's per-column operands in LDS
  half_t a[kHead], b[kHead], k[kHead], wd[kHead], r[kHead];
  half_t v[kHead];  // per state row, not per column: parked here between its arrival and its step
};

__global__ __launch_bounds__(kWave) void wkv7_f16state_kernel(int T, int C, int H, half_t* __restrict__ state,
                                                              const half_t* __restrict__ r, const half_t* __restrict__ w,
                                                              const half_t* __restrict__ w0, const half_t* __restrict__ k,
                                                              const half_t* __restrict__ v, const half_t* __restrict__ a,
                                                              const half_t* __restrict__ b, half_t* __restrict__ y,
                                                              const int* __restrict__ elapsed) {
  __shared__ __align__(16) TokenOps ops[2];
  const int bh = blockIdx.x;
  const int bi = bh / H;
  const int h = bh - bi * H;
  const int lane = threadIdx.x;
  const int c = h * kHead + lane;

  // state row `lane`: 128 bytes
  half_t* srow = state + (static_cast<int64_t>(bh) * kHead + lane) * kHead;
  half2_t S[kPairs];
#pragma unroll
  for (int q = 0; q < kPairs / 4; ++q) {
    const uint4_t t = *reinterpret_cast<const uint4_t*>(srow + 8 * q);
#pragma unroll
    for (int e = 0; e < 4; ++e) S[4 * q + e] = as_half2(t[e]);
  }

  const int phase0 = elapsed[bi] + c;
  // w0 once, not under a branch inside every step (adding 0.0f changes no decay)
  const float w0f = w0 ? h2f(w0[c]) : 0.0f;
  const int64_t tok0 = static_cast<int64_t>(bi) * T * C + c;  // this lane's element of token 0
  // token 0's operands
  {
    ops[0].a[lane] = a[tok0];
    ops[0].b[lane] = b[tok0];
    ops[0].k[lane] = k[tok0];
    ops[0].r[lane] = r[tok0];
    ops[0].wd[lane] = decay_delta16_of(h2f(w[tok0]) + w0f, phase0);
  }
  ops[0].v[lane] = v[tok0];
  // The elements of tokens t + 1 .. t + kAhead wait in registers (slot = token mod kAhead): requested one token
  // ahead only, every step would last a whole trip to memory.  Tokens past the end re-read the last one (no load
  // under a branch).
  half_t qa[kAhead], qb[kAhead], qk[kAhead], qr[kAhead], qw[kAhead], qv[kAhead];
  auto request = [&](int slot, int t) {
    const int64_t i = tok0 + static_cast<int64_t>(t < T ? t : T - 1) * C;
    qa[slot] = a[i];
    qb[slot] = b[i];
    qk[slot] = k[i];
    qr[slot] = r[i];
    qw[slot] = w[i];
    qv[slot] = v[i];
  };
#pragma unroll
  for (int u = 1; u <= kAhead; ++u) request(u % kAhead, u);
  __syncthreads();

  // One token: token t + 1's elements leave their slot for the other buffer first (nobody reads it during this
  // step), then the slot is requested again for token t + 1 + kAhead - in that order, so that the new request can
  // take the registers of the old values - and then the state step with the operands in ops[t & 1].
  auto step = [&](int t, int slot) {
    const TokenOps& cur = ops[t & 1];
    TokenOps& nxt = ops[(t + 1) & 1];
    nxt.a[lane] = qa[slot];
    nxt.b[lane] = qb[slot];
    nxt.k[lane] = qk[slot];
    nxt.r[lane] = qr[slot];
    nxt.wd[lane] = decay_delta16_of(h2f(qw[slot]) + w0f, phase0 + t + 1);
    nxt.v[lane] = qv[slot];
    __builtin_amdgcn_sched_barrier(0);
    request(slot, t + 1 + kAhead);
    __builtin_amdgcn_sched_barrier(0);
    y[tok0 + static_cast<int64_t>(t) * C] = wkv16_row_step(S, cur.a, cur.b, cur.k, cur.wd, cur.r, cur.v[lane]);
    __syncthreads();
  };
  // whole rounds of kAhead tokens as straight-line code (a loop with an exit between the steps would wait for every
  // outstanding request at its head), then the rest
  int t = 0;
  for (; t + kAhead <= T; t += kAhead) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) step(t + u, (u + 1) % kAhead);
  }
#pragma unroll
  for (int u = 0; u < kAhead - 1; ++u) {
    if (t + u < T) step(t + u, (u + 1) % kAhead);
  }

#pragma unroll
  for (int q = 0; q < kPairs / 4; ++q) {
    uint4_t t;
#pragma unroll
    for (int e = 0; e < 4; ++e) t[e] = __builtin_bit_cast(uint32_t, S[4 * q + e]);
    *reinterpret_cast<uint4_t*>(srow + 8 * q) = t;
  }
}

// ---- one token per batch row (a decode step of many rows): kk normalise / a-gate, the decay delta, the step and
// GroupNorm / bonus / gate in one launch, one wavefront per (batch row, head), four per block.  The arithmetic is that
// of kk_a_gate_kernel, wkv7_f16state_kernel (T = 1, w0 added inside) and lnx_rkvres_xg_kernel (fused_ops.hip) in
// the same order, so the result is bitwise theirs.  What differs is how the state moves: here a wavefront reads
// its head's 8 KB as eight coalesced 1 KB requests (the stand-alone kernel's lanes read one 128-byte row each, 64
// lines per request), turns them into one row per lane through a padded LDS tile, and stores the new state the same
// way back; only the wavefront itself synchronises.
constexpr int kTileLd = kHead + 8;  // halfs per tile row: 144 bytes, so that the lanes' 16-byte row reads spread over the banks

__global__ __launch_bounds__(256) void tmix16_rows_kernel(Tmix16RowsArgs p) {
  __shared__ __align__(16) half_t tile[4][kHead * kTileLd];
  __shared__ __align__(16) half_t ops[4][5][kHead];  // a~, b~, k', decay delta, r
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int64_t rh = static_cast<int64_t>(blockIdx.x) * 4 + wave;
  if (rh >= p.rows_heads) return;  // (the whole wavefront; nothing below waits for another wavefront)
  const int bi = static_cast<int>(rh / p.H);
  const int h = static_cast<int>(rh - static_cast<int64_t>(bi) * p.H);
  const int c = h * kHead + lane;
  const int64_t idx = rh * kHead + lane;

  // ---- every load first
  half_t* sbase = p.state + rh * (kHead * kHead);
  uint4_t st[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    st[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(sbase + i * 512 + lane * 8));
  const half_t k_h = p.k[idx], r_h = p.r[idx], v_h = p.v[idx], w12_h = p.w12[idx], a12_h = p.a12[idx], g_h = p.g[idx];
  const half_t kk_h = p.k_k[c], a0_h = p.a0[c], ka_h = p.k_a[c], w0_h = p.w0[c], rk_h = p.r_k[c], lnw_h = p.lnx_w[c],
               lnb_h = p.lnx_b[c];
  const int phase = p.elapsed[bi] + c;
  __builtin_amdgcn_sched_barrier(0);

  half_t* tl = tile[wave];
  const int trow = lane >> 3, tcol = (lane & 7) * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4_t*>(tl + (i * 8 + trow) * kTileLd + tcol) = st[i];

  // ---- kk normalise, a-gate, decay delta (kk_a_gate_kernel; decay_delta16 with w0 added unrounded)
  const float kv = h2f(k_h);
  const float u = kv * h2f(kk_h);
  const float total = wave_sum(u * u);
  const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
  const float kk = u * inv;
  const float av = sigmoid_f(h2f(a0_h) + h2f(a12_h));
  const float ka = h2f(ka_h);
  const half_t nk = f2h(kv * fmaf(av, ka, 1.0f - ka));
  ops[wave][0][lane] = f2h(-kk);
  ops[wave][1][lane] = f2h(kk * av);
  ops[wave][2][lane] = nk;
  ops[wave][3][lane] = decay_delta16_of(h2f(w12_h) + h2f(w0_h), phase);
  ops[wave][4][lane] = r_h;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // ---- the step on this lane's state row
  half2_t S[kPairs];
  read_pairs16(tl + lane * kTileLd, S);
  const half_t y16 = wkv16_row_step(S, ops[wave][0], ops[wave][1], ops[wave][2], ops[wave][3], ops[wave][4], v_h);
#pragma unroll
  for (int q = 0; q < kPairs / 4; ++q) {
    uint4_t t;
#pragma unroll
    for (int e = 0; e < 4; ++e) t[e] = __builtin_bit_cast(uint32_t, S[4 * q + e]);
    *reinterpret_cast<uint4_t*>(tl + lane * kTileLd + 8 * q) = t;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint4_t t = *reinterpret_cast<const uint4_t*>(tl + (i * 8 + trow) * kTileLd + tcol);
    __builtin_nontemporal_store(t, reinterpret_cast<uint4_t*>(sbase + i * 512 + lane * 8));
  }

  // ---- GroupNorm over the head, bonus, gate (lnx_rkvres_xg_kernel)
  const float yv = h2f(y16);
  const float mean = wave_sum(yv) * (1.0f / 64.0f);
  const float d = yv - mean;
  const float var = wave_sum(d * d) * (1.0f / 64.0f);
  const float rstd = rsqrtf(var + kLnxEps);
  const float rkv = wave_sum(h2f(r_h) * h2f(nk) * h2f(rk_h));
  const float o = (d * rstd * h2f(lnw_h) + h2f(lnb_h) + rkv * h2f(v_h)) * h2f(g_h);
  p.y2[idx] = f2h(o);
}

}  // namespace

int tmix16_rows_launch(hipStream_t st, const Tmix16RowsArgs& p) {
  RWKV_REQUIRE(p.rows_heads > 0 && p.H > 0, "tmix16_rows: bad shape");
  RWKV_REQUIRE(p.state && p.elapsed && p.r && p.k && p.v && p.w12 && p.a12 && p.g && p.k_k && p.a0 && p.k_a && p.w0 &&
                   p.r_k && p.lnx_w && p.lnx_b && p.y2,
               "tmix16_rows: NULL tensor");
  hipLaunchKernelGGL(tmix16_rows_kernel, dim3(static_cast<unsigned>(ceil_div(p.rows_heads, 4))), dim3(256), 0, st, p);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int wkv7_f16state_launch(hipStream_t st, int B, int T, int C, int H, half_t* state, const half_t* r, const half_t* w,
                         const half_t* w0, const half_t* k, const half_t* v, const half_t* a, const half_t* b, half_t* y,
                         const int* elapsed) {
  RWKV_REQUIRE(B > 0 && T > 0 && H > 0, "wkv7_f16state: B, T, H must be positive");
  RWKV_REQUIRE(C == H * kHead, "wkv7_f16state: C (%d) must equal H*64 (H=%d)", C, H);
  RWKV_REQUIRE(state && r && w && k && v && a && b && y && elapsed, "wkv7_f16state: NULL tensor");
  hipLaunchKernelGGL(wkv7_f16state_kernel, dim3(B * H), dim3(kWave), 0, st, T, C, H, state, r, w, w0, k, v, a, b, y, elapsed);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" int rwkv_hip_wkv7_f16state(rwkv_stream_t s, int B, int T, int C, int H, void* state, const void* r,
                                      const void* w, const void* w0, const void* k, const void* v, const void* a,
                                      const void* b, void* y, const void* elapsed) {
  return wkv7_f16state_launch(as_stream(s), B, T, C, H, static_cast<half_t*>(state), static_cast<const half_t*>(r),
                              static_cast<const half_t*>(w), static_cast<const half_t*>(w0), static_cast<const half_t*>(k),
                              static_cast<const half_t*>(v), static_cast<const half_t*>(a), static_cast<const half_t*>(b),
                              static_cast<half_t*>(y), static_cast<const int*>(elapsed));
}
