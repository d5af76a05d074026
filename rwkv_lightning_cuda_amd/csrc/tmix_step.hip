// Decode-step (T == 1) time-mix core, one workgroup per (batch row, head): everything between the r/k/v
// projections and the output projection in a single launch.
//
// Fuses, with the reference's fp16 rounding points kept in registers:
//   LoRA rank-out x4 (+tanh / sigmoid, v-residual gate) ... cuda/rwkv7_v3a_ops.cu:1027-1130
//   w_raw = w12 + w0 .................................... cuda/rwkv7_fast_ops_fp16.cu:462-477
//   kk normalise, a-gate, k' ............................ cuda/rwkv7_fast_ops_fp16.cu:129-172
//   WKV7 state update for one token ..................... cuda/rwkv7_wkv_fp32_v2.cu:134-174 (small_warp kernel)
//   per-head GroupNorm + bonus + gate ................... cuda/rwkv7_fast_ops_fp16.cu:174-237
// The reference launches seven kernels for this; at batch 1 each is latency-bound, so one launch that
// issues all of its loads up front (state rows, LoRA rows, vectors) costs about as much as one of them.
//
// Layout: 1024 threads = 64 channels x 16 lanes.  Every global load of the launch is issued before the first
// use (one memory round trip): lane q of channel i loads its 16-byte slice of state row i (the 16 lanes of
// a row read 256 contiguous bytes) and up to four 8-element chunks (q, q+16, ...) of each of the channel's
// LoRA rows; the 16 lanes of a channel are one DPP row, so row sums take four DPP adds.  The twelve per-channel
// scalars (projections, biases, norm weights) are loaded by the first wavefront only, lane = channel: a load
// instruction costs the CU's address unit the same 16 clocks whether it fetches 2 or 16 bytes per lane, and with
// every wavefront fetching its own copies the scalars were more than half of the launch's load instructions.
// That wavefront also does everything that is per channel - kk normalisation, a-gate, decay, v-residual gate,
// and at the end GroupNorm, bonus and gate, its three sums over the head taken inside the wavefront - between the
// block-wide phases (rank-outs, state update) that need all 1024 threads; four barriers in all.
//
// A block's loads (123 KB at the 7.2B shape, 61 KB of them the g rank-out rows) arrive at the rate one CU can
// take in, about 50 GB/s, and only B*H CUs are at work.  In split mode the g rank-out therefore runs in B*H
// further blocks of the same launch, and the gate is applied by the consumer of the output (see TmixStepArgs).
#include "wkv7_f16state.h"

namespace rwkv {

constexpr int kStepMaxR = 512;
constexpr int kStepLanes = 16;                       // lanes per channel
constexpr int kStepThreads = kHead * kStepLanes;     // 1024
constexpr int kStepChunks = kStepMaxR / (8 * kStepLanes);  // 4

// A channel's LoRA row as the 16 lanes of the channel hold it: lane q has the 8-element chunks q, q + 16, ... of
// the row, one per round of 128 elements.  Whether a round exists is the same for the whole wavefront (a scalar
// branch); inside the last round a lane past the end of the row re-reads the row's last chunk, which then meets
// zeros of the hidden vector.  Nothing here is predicated per lane or merged with a default value: both make the
// compiler copy a loaded register inside the branch, and that copy waits for every load issued so far.
struct LoraRow {
  half8_t w[kStepChunks];
};

__device__ __forceinline__ void lora_row_load(LoraRow& row, const half_t* __restrict__ wrow, int R, int q) {
#pragma unroll
  for (int ii = 0; ii < kStepChunks; ++ii) {
    if (ii * (8 * kStepLanes) < R) {
      const int r0 = (q + kStepLanes * ii) * 8;
      row.w[ii] = *reinterpret_cast<const half8_t*>(wrow + (r0 < R ? r0 : R - 8));
    }
  }
}

// dot of a channel's LoRA row with the activated hidden vector (zeros from R up to the end of its last round);
// all 16 lanes of the channel get the sum
__device__ __forceinline__ float lora_row_dot(const LoraRow& row, const float* __restrict__ hs, int R, int q) {
  float acc = 0.0f;
#pragma unroll
  for (int ii = 0; ii < kStepChunks; ++ii) {
    if (ii * (8 * kStepLanes) < R) {
      const int r0 = (q + kStepLanes * ii) * 8;
      const float4_t h0 = *reinterpret_cast<const float4_t*>(hs + r0);
      const float4_t h1 = *reinterpret_cast<const float4_t*>(hs + r0 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = fmaf(h0[e], h2f(row.w[ii][e]), acc);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = fmaf(h1[e], h2f(row.w[ii][4 + e]), acc);
    }
  }
  return row16_sum(acc);
}

// Element `tid` of a hidden vector, raw, for the wavefronts that cover [0, roundup(R, 128)); others get nothing.
__device__ __forceinline__ void hidden_load(half_t& raw, const half_t* __restrict__ hid, int R, int wave, int tid) {
  if (wave * 64 < R) raw = hid[tid < R ? tid : R - 1];
}
// Keeps the uses of a loaded value below this point: the compiler otherwise moves the conversion up into the branch
// of the load, where it waits for every load the wavefront has issued so far before the next one is issued.
__device__ __forceinline__ void use_below(half_t& raw) {
  unsigned v = __builtin_bit_cast(unsigned short, raw);
  asm volatile("" : "+v"(v));
  raw = __builtin_bit_cast(half_t, static_cast<unsigned short>(v));
}
// activation (0 none, 1 tanh, 2 sigmoid) into LDS; zeros from R to the end of the last round of 128
template <int ACT>
__device__ __forceinline__ void hidden_store(float* __restrict__ hs, half_t raw, int R, int wave, int tid) {
  if (wave * 64 < ((R + 127) & ~127)) {
    float v = 0.0f;
    if (wave * 64 < R) {
      v = h2f(raw);
      if (ACT == 1) v = tanh_f(v);
      if (ACT == 2) v = sigmoid_f(v);
      if (tid >= R) v = 0.0f;
    }
    hs[tid] = v;
  }
}

// F16: the WKV state is fp16 and the step follows the fp16-state recurrence (wkv7_f16state.h): the first wavefront
// holds the head's 64 state rows, one per lane, and does the step itself between its per-channel work and the
// GroupNorm - the other wavefronts are done after the rank-outs, two barriers in all.
template <bool F16>
__global__ __launch_bounds__(kStepThreads) void tmix_step_kernel(TmixStepArgs p) {
  __shared__ __align__(16) half_t ops16[5][kHead];  // fp16-state mode: a~, b~, k', decay delta, r
  __shared__ __align__(16) float hs[4][kStepMaxR];  // activated LoRA hidden vectors: w, a, g, v
  __shared__ __align__(16) float lo[4][kHead];      // rank-out results per channel: w12, a12, g, v-gate logit
  __shared__ __align__(16) float vec[6][kHead];     // WKV operands r, d, k', a~, b~ and the mixed v
  __shared__ float yv[kHead];                       // y of the step, rounded to fp16

  const bool split = p.gate_out != nullptr;
  const int n_heads = p.B * p.H;
  const bool gate_block = static_cast<int>(blockIdx.x) >= n_heads;
  const int bh = gate_block ? blockIdx.x - n_heads : blockIdx.x;
  const int bi = bh / p.H;
  const int h = bh - bi * p.H;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int i = tid / kStepLanes;  // channel within the head / state row
  const int q = tid % kStepLanes;
  const int c = h * kHead + i;
  const int64_t row = static_cast<int64_t>(bi) * p.C;

  if (gate_block) {
    // the g rank-out of the head's 64 channels, nothing else
    LoraRow g2;
    lora_row_load(g2, p.g2 + static_cast<int64_t>(c) * p.Rg, p.Rg, q);
    half_t hraw;
    hidden_load(hraw, p.hg + static_cast<int64_t>(bi) * p.Rg, p.Rg, wave, tid);
    __builtin_amdgcn_sched_barrier(0);
    use_below(hraw);
    hidden_store<2>(hs[2], hraw, p.Rg, wave, tid);
    __syncthreads();
    const float gch = lora_row_dot(g2, hs[2], p.Rg, q);
    if (q == 0) p.gate_out[row + c] = f2h(gch);
    return;
  }

  // ---- all global loads up front
  float* srow = nullptr;
  float4_t S = {0.0f, 0.0f, 0.0f, 0.0f};
  half_t* srow16 = nullptr;
  half2_t S16[kPairs16];
  int phase = 0;
  if constexpr (F16) {
    if (wave == 0) {  // state row `lane` of the head: 128 bytes
      srow16 = p.state16 + (static_cast<int64_t>(bh) * kHead + lane) * kHead;
#pragma unroll
      for (int g = 0; g < kPairs16 / 4; ++g) {
        const uint4_t t = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(srow16 + 8 * g));
#pragma unroll
        for (int e = 0; e < 4; ++e) S16[4 * g + e] = as_half2(t[e]);
      }
      phase = p.elapsed[bi];
    }
  } else {
    srow = p.state + (static_cast<int64_t>(bh) * kHead + i) * kHead + 4 * q;
    S = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(srow));
  }
  LoraRow w2, a2, g2, v2;
  lora_row_load(w2, p.w2 + static_cast<int64_t>(c) * p.Rw, p.Rw, q);
  lora_row_load(a2, p.a2 + static_cast<int64_t>(c) * p.Ra, p.Ra, q);
  if (!split) lora_row_load(g2, p.g2 + static_cast<int64_t>(c) * p.Rg, p.Rg, q);
  if (p.hv) lora_row_load(v2, p.v2 + static_cast<int64_t>(c) * p.Rv, p.Rv, q);
  // Activated hidden vectors and per-channel scalars: only the loads here, as raw fp16 - a conversion next to its
  // load would make the wavefront wait for everything it has requested so far before it requests the rest (loads
  // return in order), one trip to memory after another.  The scalars: first wavefront, lane = channel.
  half_t hw_raw, ha_raw, hg_raw, hv_raw;
  hidden_load(hw_raw, p.hw + static_cast<int64_t>(bi) * p.Rw, p.Rw, wave, tid);
  hidden_load(ha_raw, p.ha + static_cast<int64_t>(bi) * p.Ra, p.Ra, wave, tid);
  if (!split) hidden_load(hg_raw, p.hg + static_cast<int64_t>(bi) * p.Rg, p.Rg, wave, tid);
  if (p.hv) hidden_load(hv_raw, p.hv + static_cast<int64_t>(bi) * p.Rv, p.Rv, wave, tid);
  const half_t hzero = static_cast<half_t>(0.0f);
  half_t kv_h = hzero, rv_h = hzero, vv_h = hzero, kkw_h = hzero, a0_h = hzero, ka_h = hzero, w0_h = hzero, rk_h = hzero,
         lnw_h = hzero, lnb_h = hzero, v0_h = hzero, vf_h = hzero, shift_h = hzero;
  const int cl = h * kHead + lane;  // the first wavefront's channel
  if (wave == 0) {
    kv_h = p.k[row + cl];
    rv_h = p.r[row + cl];
    vv_h = p.v[row + cl];
    kkw_h = p.k_k[cl];
    a0_h = p.a0[cl];
    ka_h = p.k_a[cl];
    w0_h = p.w0[cl];
    rk_h = p.r_k[cl];
    lnw_h = p.lnx_w[cl];
    lnb_h = p.lnx_b[cl];
    if (p.hv) {
      v0_h = p.v0[cl];
      vf_h = p.v_first[row + cl];
    }
    if (p.shift_dst) shift_h = p.shift_src[row + cl];
  }
  __builtin_amdgcn_sched_barrier(0);
  use_below(hw_raw);
  use_below(ha_raw);
  if (!split) use_below(hg_raw);
  if (p.hv) use_below(hv_raw);

  hidden_store<1>(hs[0], hw_raw, p.Rw, wave, tid);
  hidden_store<0>(hs[1], ha_raw, p.Ra, wave, tid);
  if (!split) hidden_store<2>(hs[2], hg_raw, p.Rg, wave, tid);
  if (p.hv) hidden_store<0>(hs[3], hv_raw, p.Rv, wave, tid);
  const float kv = h2f(kv_h), rv = h2f(rv_h), vv = h2f(vv_h), kkw = h2f(kkw_h), a0 = h2f(a0_h), ka = h2f(ka_h),
              w0 = h2f(w0_h), rk = h2f(rk_h), lnw = h2f(lnw_h), lnb = h2f(lnb_h), v0 = h2f(v0_h), vf = h2f(vf_h);
  __syncthreads();

  // ---- LoRA rank-outs for channel i (fp32 sums over the 16 lanes)
  {
    const float w12 = round_h(lora_row_dot(w2, hs[0], p.Rw, q));
    const float a12 = round_h(lora_row_dot(a2, hs[1], p.Ra, q));
    const float gch = split ? 1.0f : round_h(lora_row_dot(g2, hs[2], p.Rg, q));
    const float vdot = p.hv ? lora_row_dot(v2, hs[3], p.Rv, q) : 0.0f;
    if (q == 0) {
      lo[0][i] = w12;
      lo[1][i] = a12;
      lo[2][i] = gch;
      lo[3][i] = vdot;
    }
  }
  __syncthreads();

  // ---- per channel, first wavefront: v-residual gate, kk normalise over the head, a-gate, decay
  float v_use = vv, k2 = 0.0f, gch = 0.0f;
  if constexpr (F16) {
    if (wave != 0) return;
  }
  if (wave == 0) {
    const float w12 = lo[0][lane];
    const float a12 = lo[1][lane];
    gch = lo[2][lane];
    if (p.hv) {
      const float gate = sigmoid_f(v0 + lo[3][lane]);
      v_use = round_h(vv + (vf - vv) * gate);
    } else if (p.v_first_out) {
      p.v_first_out[row + cl] = f2h(vv);  // layer 0: v_first = v
    }
    const float u = kv * kkw;
    const float total = wave_sum_uniform(u * u);
    const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
    const float kk = u * inv;
    const float av = sigmoid_f(a0 + a12);
    k2 = round_h(kv * fmaf(av, ka, 1.0f - ka));
    if constexpr (F16) {
      // the operands as the fp16 tensors the stand-alone kernels exchange, then the step on this lane's state row
      ops16[0][lane] = f2h(-kk);
      ops16[1][lane] = f2h(kk * av);
      ops16[2][lane] = f2h(k2);
      ops16[3][lane] = decay_delta16_of(w12 + w0, phase + cl);  // (w12 + w0 unrounded: a single-token call)
      ops16[4][lane] = f2h(rv);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const half_t y16 = wkv16_row_step(S16, ops16[0], ops16[1], ops16[2], ops16[3], ops16[4], f2h(v_use));
#pragma unroll
      for (int g = 0; g < kPairs16 / 4; ++g) {
        uint4_t t;
#pragma unroll
        for (int e = 0; e < 4; ++e) t[e] = __builtin_bit_cast(uint32_t, S16[4 * g + e]);
        __builtin_nontemporal_store(t, reinterpret_cast<uint4_t*>(srow16 + 8 * g));
      }
      const float yy = h2f(y16);
      const float mean = wave_sum_uniform(yy) * (1.0f / 64.0f);
      const float rkv = wave_sum_uniform(rv * k2 * rk);
      const float dlt = yy - mean;
      const float var = wave_sum_uniform(dlt * dlt) * (1.0f / 64.0f);
      const float rstd = rsqrtf(var + kLnxEps);
      if (p.shift_dst) p.shift_dst[row + cl] = shift_h;
      const float pre = dlt * rstd * lnw + lnb + rkv * v_use;
      if (split) {
        p.y2_pre[row + cl] = pre;
      } else {
        p.y2[row + cl] = f2h(pre * gch);
      }
      return;
    }
    const float wraw = round_h(w12 + w0);
    vec[0][lane] = rv;
    vec[1][lane] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
    vec[2][lane] = k2;
    vec[3][lane] = round_h(-kk);
    vec[4][lane] = round_h(kk * av);
    vec[5][lane] = v_use;
  }
  __syncthreads();

  // ---- WKV step on row i, this lane's 4 columns
  {
    const int j = 4 * q;
    const float vi = vec[5][i];
    const float4_t a4 = *reinterpret_cast<const float4_t*>(&vec[3][j]);
    float sa = S.x * a4.x;
    sa = fmaf(S.y, a4.y, sa);
    sa = fmaf(S.z, a4.z, sa);
    sa = fmaf(S.w, a4.w, sa);
    sa = row16_sum(sa);
    const float4_t d4 = *reinterpret_cast<const float4_t*>(&vec[1][j]);
    const float4_t k4 = *reinterpret_cast<const float4_t*>(&vec[2][j]);
    const float4_t b4 = *reinterpret_cast<const float4_t*>(&vec[4][j]);
    const float4_t r4 = *reinterpret_cast<const float4_t*>(&vec[0][j]);
    S.x = fmaf(S.x, d4.x, fmaf(sa, b4.x, k4.x * vi));
    S.y = fmaf(S.y, d4.y, fmaf(sa, b4.y, k4.y * vi));
    S.z = fmaf(S.z, d4.z, fmaf(sa, b4.z, k4.z * vi));
    S.w = fmaf(S.w, d4.w, fmaf(sa, b4.w, k4.w * vi));
    __builtin_nontemporal_store(S, reinterpret_cast<float4_t*>(srow));
    float yy = S.x * r4.x;
    yy = fmaf(S.y, r4.y, yy);
    yy = fmaf(S.z, r4.z, yy);
    yy = fmaf(S.w, r4.w, yy);
    yy = round_h(row16_sum(yy));  // the reference stores y as fp16 before the GroupNorm kernel reads it
    if (q == 0) yv[i] = yy;
  }
  __syncthreads();

  // ---- per-head GroupNorm (two-pass), bonus term, gate: first wavefront, sums inside the wavefront
  if (wave == 0) {
    const float yy = yv[lane];
    const float mean = wave_sum_uniform(yy) * (1.0f / 64.0f);
    const float rkv = wave_sum_uniform(rv * k2 * rk);
    const float dlt = yy - mean;
    const float var = wave_sum_uniform(dlt * dlt) * (1.0f / 64.0f);
    const float rstd = rsqrtf(var + kLnxEps);
    // the LN output that the r/k/v launch computed in its prologue becomes the shift row of the state (that
    // launch could not store it itself: other blocks of it were still reading the old row)
    if (p.shift_dst) p.shift_dst[row + cl] = shift_h;
    const float pre = dlt * rstd * lnw + lnb + rkv * v_use;
    if (split) {
      p.y2_pre[row + cl] = pre;
    } else {
      p.y2[row + cl] = f2h(pre * gch);
    }
  }
}

int tmix_step_launch(hipStream_t st, const TmixStepArgs& p) {
  RWKV_REQUIRE(p.B > 0 && p.H > 0 && p.C == p.H * kHead, "tmix_step: bad shape");
  RWKV_REQUIRE(p.Rw % 8 == 0 && p.Ra % 8 == 0 && p.Rg % 8 == 0 && p.Rv % 8 == 0 && p.Rw <= kStepMaxR &&
                   p.Ra <= kStepMaxR && p.Rg <= kStepMaxR && p.Rv <= kStepMaxR,
               "tmix_step: LoRA ranks must be multiples of 8, at most %d", kStepMaxR);
  RWKV_REQUIRE((p.gate_out == nullptr) == (p.y2_pre == nullptr), "tmix_step: split mode needs both y2_pre and gate_out");
  RWKV_REQUIRE((p.state != nullptr) != (p.state16 != nullptr), "tmix_step: exactly one of the fp32 and the fp16 state");
  RWKV_REQUIRE(p.state16 == nullptr || p.elapsed != nullptr, "tmix_step: the fp16 state needs the elapsed counters");
  const int blocks = p.B * p.H * (p.gate_out ? 2 : 1);
  if (p.state16) {
    hipLaunchKernelGGL(tmix_step_kernel<true>, dim3(blocks), dim3(kStepThreads), 0, st, p);
  } else {
    hipLaunchKernelGGL(tmix_step_kernel<false>, dim3(blocks), dim3(kStepThreads), 0, st, p);
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv
