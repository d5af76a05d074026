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
// gfx950 layout of the sequence kernel: a block per (batch row, head); one, two or four lanes share a state row and
// hold its 64 values as half2 pairs in registers for the whole call (v_pk_fma_f16 does both columns of a pair).  The
// five per-column vectors of a token (a, b, k, decay delta, r) are the same for every row: a wavefront of its own
// fetches them some tokens ahead, lane c element c of each, converts the decay logit and drops them into LDS, from
// where the wavefronts that own the state read them back as 16-byte pieces.  The state is read and written once
// per call, 16 bytes per lane and instruction.  Details at the kernel.
#include "wkv7_f16state.h"

namespace rwkv {

namespace {

constexpr int kPairs = kPairs16;
constexpr int kAhead = 4;  // tokens whose operands are in flight from memory
constexpr int kRing = 4;   // tokens whose operands have a place in LDS

struct TokenOps {  // one token's per-column operands in LDS
  half_t a[kHead], b[kHead], k[kHead], wd[kHead], r[kHead];
  half_t v[kHead];  // per state row, not per column: parked here between its arrival and its step
};

// The block's wavefronts meet once per token.  LDS only: what they have in flight to or from memory (the feeder's
// loads of later tokens, the others' stores of y) does not have to land first.
__device__ __forceinline__ void token_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Lanes in groups of LPR (2 or 4): every lane takes the value of its left neighbour in the group (the first keeps
// its own) / of the group's last lane.  DPP quad_perm, two bits per lane of a quad.
template <int LPR>
__device__ __forceinline__ half2_t group_from_left(half2_t x) {
  constexpr int kCtrl = LPR == 4 ? (0 | 0 << 2 | 1 << 4 | 2 << 6) : (0 | 0 << 2 | 2 << 4 | 2 << 6);
  const int xi = __builtin_bit_cast(int, x);  // (also as the value of disabled lanes - there are none - so that none is made up)
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_update_dpp(xi, xi, kCtrl, 0xf, 0xf, false));
}
template <int LPR>
__device__ __forceinline__ half2_t group_from_last(half2_t x) {
  constexpr int kCtrl = LPR == 4 ? (3 | 3 << 2 | 3 << 4 | 3 << 6) : (1 | 1 << 2 | 3 << 4 | 3 << 6);
  const int xi = __builtin_bit_cast(int, x);
  return __builtin_bit_cast(half2_t, __builtin_amdgcn_update_dpp(xi, xi, kCtrl, 0xf, 0xf, false));
}

// LPR + 1 wavefronts per (batch row, head); LPR = lanes per state row, 1, 2 or 4.
//
// A wavefront that is alone on its SIMD issues one instruction every four cycles whatever the instruction is, so
// everything that is not the recurrence itself is taken off the wavefronts that own the state: the last wavefront
// (the feeder) fetches the operands of token t + 2 + kAhead, converts the decay logit of token t + 2 and drops that
// token's operands into a ring of kRing LDS buffers while the others run token t from the ring.
//
// LPR = 1: one wavefront owns the head, lane = state row (32 pairs): 160 packed FMAs, 40 16-byte LDS broadcasts and
// one store per token.  LPR = 4 (while the grid leaves SIMDs idle): four wavefronts own sixteen rows each, and four
// neighbouring lanes share a row, sixteen columns each.  The two chains still run over the pairs in order - all
// lanes run every quarter of a chain on their own columns, the running value moves one lane to the right between
// the quarters (DPP), and only what has come through lanes 0, 1, 2, 3 in turn is used, so every sum sees the same
// operations in the same order - but the update, the LDS reads and the registers per lane are a quarter: a token
// costs a wavefront 64 + 24 packed FMAs instead of 160.  LPR = 2 likewise with halves (64 + 48).  (The four
// wavefronts together issue twice the instructions of the one: where every SIMD has a head of its own, LPR = 1 is
// the faster one.)
template <int LPR>
__global__ __launch_bounds__((LPR + 1) * kWave) void wkv7_f16state_kernel(int T, int C, int H, half_t* __restrict__ state,
                                                                          const half_t* __restrict__ r, const half_t* __restrict__ w,
                                                                          const half_t* __restrict__ w0, const half_t* __restrict__ k,
                                                                          const half_t* __restrict__ v, const half_t* __restrict__ a,
                                                                          const half_t* __restrict__ b, half_t* __restrict__ y,
                                                                          const int* __restrict__ elapsed) {
  static_assert(LPR == 1 || LPR == 2 || LPR == 4, "lanes per state row: 1, 2 or 4");
  constexpr int NP = kPairs / LPR;  // pairs of a row per lane
  __shared__ __align__(16) TokenOps ops[kRing];
  const int bh = blockIdx.x;
  const int bi = bh / H;
  const int h = bh - bi * H;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  // Element c of token t of this head sits (t * C + c) * 2 bytes behind a base that is the same for the whole
  // block: one 32-bit offset per token serves all six loads or the store (the launcher checks that it fits).
  const int64_t head0 = static_cast<int64_t>(bi) * T * C + h * kHead;
  const unsigned row_bytes = static_cast<unsigned>(C) * 2u;

  if (wave == LPR) {  // the feeder: lane = column (and row, for v)
    const unsigned lane2 = static_cast<unsigned>(lane) * 2u;
    const int c = h * kHead + lane;
    const half_t* pr = r + head0;
    const half_t* pw = w + head0;
    const half_t* pk = k + head0;
    const half_t* pv = v + head0;
    const half_t* pa = a + head0;
    const half_t* pb = b + head0;
    const int phase0 = elapsed[bi] + c;
    // w0 once, not under a branch inside every step (adding 0.0f changes no decay)
    const float w0f = w0 ? h2f(w0[c]) : 0.0f;
    auto at = [](const half_t* base, unsigned byte_off) {
      return *reinterpret_cast<const half_t*>(reinterpret_cast<const char*>(base) + byte_off);
    };
    // The elements of kAhead tokens wait in registers (slot = token mod kAhead): requested one token ahead only,
    // every step would last a whole trip to memory.  Tokens past the end re-read the last one (no load under a
    // branch) and land in ring places nobody reads any more.
    half_t qa[kAhead], qb[kAhead], qk[kAhead], qr[kAhead], qw[kAhead], qv[kAhead];
    auto request = [&](int slot, int t) {
      const unsigned off = lane2 + static_cast<unsigned>(t < T ? t : T - 1) * row_bytes;
      qa[slot] = at(pa, off);
      qb[slot] = at(pb, off);
      qk[slot] = at(pk, off);
      qr[slot] = at(pr, off);
      qw[slot] = at(pw, off);
      qv[slot] = at(pv, off);
    };
    auto place = [&](int slot, int t) {  // token t from its slot into its place in the ring
      TokenOps& o = ops[t & (kRing - 1)];
      o.a[lane] = qa[slot];
      o.b[lane] = qb[slot];
      o.k[lane] = qk[slot];
      o.r[lane] = qr[slot];
      o.wd[lane] = decay_delta16_of(h2f(qw[slot]) + w0f, phase0 + t);
      o.v[lane] = qv[slot];
    };
    request(0, 0);
    request(1, 1);
    place(0, 0);
    place(1, 1);
#pragma unroll
    for (int u = 0; u < kAhead; ++u) request((2 + u) % kAhead, 2 + u);
    token_barrier();
    // step t: token t + 2 into the ring (its place was token t - 2's, which the others left two meetings ago), its
    // slot requested again for token t + 2 + kAhead
    auto step = [&](int t, int slot) {
      place(slot, t + 2);
      __builtin_amdgcn_sched_barrier(0);
      request(slot, t + 2 + kAhead);
      token_barrier();
    };
    // whole rounds of kAhead tokens as straight-line code (a loop with an exit between the steps would wait for
    // every outstanding request at its head), then the rest
    int t = 0;
    for (; t + kAhead <= T; t += kAhead) {
#pragma unroll
      for (int u = 0; u < kAhead; ++u) step(t + u, (2 + u) % kAhead);
    }
#pragma unroll
    for (int u = 0; u < kAhead - 1; ++u) {
      if (t + u < T) step(t + u, (2 + u) % kAhead);
    }
    return;
  }

  // ---- the wavefronts that own the state: this lane's NP pairs of its row
  const int row = wave * (kWave / LPR) + lane / LPR;
  const int col0 = (lane % LPR) * (2 * NP);
  half_t* srow = state + (static_cast<int64_t>(bh) * kHead + row) * kHead + col0;
  half_t* py = y + head0;
  const unsigned row2 = static_cast<unsigned>(row) * 2u;
  auto read_part = [&](const half_t* vec, half2_t(&dst)[NP]) {  // this lane's columns of a per-column vector
#pragma unroll
    for (int q = 0; q < NP / 4; ++q) {
      const uint4_t t = *reinterpret_cast<const uint4_t*>(vec + col0 + 8 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[4 * q + e] = as_half2(t[e]);
    }
  };
  half2_t S[NP];
  read_part(srow - col0, S);
  token_barrier();

  // One token, in an order that leaves no packed FMA right behind the one it depends on (the hardware wants an idle
  // issue slot there, which costs a wavefront as much as an instruction):
  //   - the chain over a of this token runs interleaved with the chain over r of the token BEFORE (both read the
  //     state between the two tokens; r of that token stays in registers), whose y is stored one step late;
  //   - the update runs over eight pairs at a time, one of its three FMAs for all eight before the next.
  // Every value sees the same operations in the same order as in wkv16_row_step.
  // Where the LDS reads sit: the first half of b / k / decay delta of token t is requested ahead of the two chains
  // of step t, the second half, r of token t and a of token t + 1 right after them (r and a into the registers the
  // chains have just finished with; LPR = 1: a half way through the update, so that the step fits the 256
  // registers): each is there by the time it is used.
  half2_t r_prev[NP], a_cur[NP];
#pragma unroll
  for (int j = 0; j < NP; ++j) r_prev[j] = half2_t{static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
  read_part(ops[0].a, a_cur);
  auto step = [&](int t) {
    const TokenOps& cur = ops[t & (kRing - 1)];
    const TokenOps& nxt = ops[(t + 1) & (kRing - 1)];
    const half_t v_cur = cur.v[row];
    half2_t bv[NP], kv[NP], wv[NP];
    auto read_bkw = [&](int q) {  // pairs 4q .. 4q + 3 of this lane's b, k and decay delta
      const uint4_t tb = *reinterpret_cast<const uint4_t*>(cur.b + col0 + 8 * q);
      const uint4_t tk = *reinterpret_cast<const uint4_t*>(cur.k + col0 + 8 * q);
      const uint4_t tw = *reinterpret_cast<const uint4_t*>(cur.wd + col0 + 8 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bv[4 * q + e] = as_half2(tb[e]);
        kv[4 * q + e] = as_half2(tk[e]);
        wv[4 * q + e] = as_half2(tw[e]);
      }
    };
#pragma unroll
    for (int q = 0; q < NP / 8; ++q) read_bkw(q);
    __builtin_amdgcn_sched_barrier(0);
    half2_t sa2 = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
    half2_t y2 = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
#pragma unroll
    for (int part = 0; part < LPR; ++part) {
      if (part > 0) {  // what the lane to the left has summed over its columns goes on over this lane's
        sa2 = group_from_left<LPR>(sa2);
        y2 = group_from_left<LPR>(y2);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        sa2 = pk_fma16(a_cur[j], S[j], sa2);
        y2 = pk_fma16(S[j], r_prev[j], y2);
        __builtin_amdgcn_sched_barrier(0);  // (left alone, the compiler may run one chain after the other)
      }
    }
    if constexpr (LPR > 1) {  // the sums over all 64 columns are in the last lane of the four
      sa2 = group_from_last<LPR>(sa2);
      y2 = group_from_last<LPR>(y2);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = NP / 8; q < NP / 4; ++q) read_bkw(q);
    read_part(cur.r, r_prev);
    if constexpr (LPR > 1) read_part(nxt.a, a_cur);
    // y of token t - 1 (at t = 0: a zero into y of token 0, which the next step overwrites); the lanes that share
    // a row store the same value
    *reinterpret_cast<half_t*>(reinterpret_cast<char*>(py) + (row2 + static_cast<unsigned>(t > 0 ? t - 1 : 0) * row_bytes)) =
        y2[0] + y2[1];
    const half_t sa = sa2[0] + sa2[1];
    const half2_t sa_b = {sa, sa};
    const half2_t vv = {v_cur, v_cur};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < NP / 8; ++g) {
      half2_t u[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = pk_fma16(sa_b, bv[8 * g + e], S[8 * g + e]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = pk_fma16(kv[8 * g + e], vv, u[e]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int e = 0; e < 8; ++e) S[8 * g + e] = pk_fma16(S[8 * g + e], wv[8 * g + e], u[e]);
      if (LPR == 1 && g == 1) read_part(nxt.a, a_cur);  // (registers: half of b / k / decay delta are done with)
      __builtin_amdgcn_sched_barrier(0);
    }
    token_barrier();
  };
  int t = 0;
  for (; t + kAhead <= T; t += kAhead) {
#pragma unroll
    for (int u = 0; u < kAhead; ++u) step(t + u);
  }
#pragma unroll
  for (int u = 0; u < kAhead - 1; ++u) {
    if (t + u < T) step(t + u);
  }
  {  // y of the last token
    half2_t y2 = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
#pragma unroll
    for (int part = 0; part < LPR; ++part) {
      if (part > 0) y2 = group_from_left<LPR>(y2);
#pragma unroll
      for (int j = 0; j < NP; ++j) y2 = pk_fma16(S[j], r_prev[j], y2);
    }
    if constexpr (LPR > 1) y2 = group_from_last<LPR>(y2);
    *reinterpret_cast<half_t*>(reinterpret_cast<char*>(py) + (row2 + static_cast<unsigned>(T - 1) * row_bytes)) = y2[0] + y2[1];
  }

#pragma unroll
  for (int q = 0; q < NP / 4; ++q) {
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
  // (this wavefront has its SIMD nearly to itself at the batch sizes this kernel serves: sums without LDS round
  // trips, in the stand-alone kernels' order and with their fused first level)
  const float total = wave_sum_dpp_of_product(u, u);
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
  const float mean = wave_sum_dpp(yv) * (1.0f / 64.0f);
  const float d = yv - mean;
  const float var = wave_sum_dpp_of_product(d, d) * (1.0f / 64.0f);
  const float rstd = rsqrtf(var + kLnxEps);
  float rk2;
  {
#pragma clang fp contract(off)
    rk2 = h2f(r_h) * h2f(nk);
  }
  const float rkv = wave_sum_dpp_of_product(rk2, h2f(rk_h));
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
  RWKV_REQUIRE(static_cast<int64_t>(T) * C < (int64_t{1} << 31), "wkv7_f16state: T * C = %lld does not fit the kernel's 32-bit byte offsets",
               static_cast<long long>(static_cast<int64_t>(T) * C));
  // four (two) lanes per state row while that leaves no SIMD with more than one state-owning wavefront
  const int64_t heads = static_cast<int64_t>(B) * H;
  const int cus = device_cu_count();
  if (heads <= cus) {
    hipLaunchKernelGGL(wkv7_f16state_kernel<4>, dim3(B * H), dim3(5 * kWave), 0, st, T, C, H, state, r, w, w0, k, v, a, b, y, elapsed);
  } else if (heads <= 2 * cus) {
    hipLaunchKernelGGL(wkv7_f16state_kernel<2>, dim3(B * H), dim3(3 * kWave), 0, st, T, C, H, state, r, w, w0, k, v, a, b, y, elapsed);
  } else {
    hipLaunchKernelGGL(wkv7_f16state_kernel<1>, dim3(B * H), dim3(2 * kWave), 0, st, T, C, H, state, r, w, w0, k, v, a, b, y, elapsed);
  }
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
