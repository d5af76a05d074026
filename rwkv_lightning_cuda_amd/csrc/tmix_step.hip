// Decode-step (T == 1) time-mix core, one workgroup per head and one, two or four batch rows: everything between
// the r/k/v projections and the output projection in a single launch.
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
// scalars (projections, biases, norm weights) are loaded by one wavefront per batch row only, lane = channel: a load
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
// (The row's registers are copied by an asm statement first: called in a loop over batch rows, the fp16 -> fp32
// conversions would otherwise be taken out of the loop and kept, twice the registers of the row itself.  A copy, not
// an in-place pass: a row register rewritten under the round's condition becomes a value merged at the end of a
// branch, and such a value is copied right after its load, behind a wait for every load issued so far.)
__device__ __forceinline__ float lora_row_dot(const LoraRow& row, const float* __restrict__ hs, int R, int q) {
  float acc = 0.0f;
#pragma unroll
  for (int ii = 0; ii < kStepChunks; ++ii) {
    if (ii * (8 * kStepLanes) < R) {
      const uint4_t raw = __builtin_bit_cast(uint4_t, row.w[ii]);
      uint4_t cp;
      asm volatile("v_mov_b32 %0, %4\n\tv_mov_b32 %1, %5\n\tv_mov_b32 %2, %6\n\tv_mov_b32 %3, %7"
                   : "=&v"(cp.x), "=&v"(cp.y), "=&v"(cp.z), "=&v"(cp.w)
                   : "v"(raw.x), "v"(raw.y), "v"(raw.z), "v"(raw.w));
      const half8_t w = __builtin_bit_cast(half8_t, cp);
      const int r0 = (q + kStepLanes * ii) * 8;
      const float4_t h0 = *reinterpret_cast<const float4_t*>(hs + r0);
      const float4_t h1 = *reinterpret_cast<const float4_t*>(hs + r0 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = fmaf(h0[e], h2f(w[e]), acc);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = fmaf(h1[e], h2f(w[4 + e]), acc);
    }
  }
  return row16_sum(acc);
}

// Element `tid` of a hidden vector, raw, for the wavefronts that cover [0, roundup(R, 128)); others get nothing.
// Loaded as the aligned 32-bit pair that holds it (R is even), the half picked at the store below: a 16-bit load's
// widening is an instruction of its own that ends up next to the load, with a wait.
__device__ __forceinline__ void hidden_load(unsigned& raw, const half_t* __restrict__ hid, int R, int wave, int tid) {
  if (wave * 64 < R) raw = *reinterpret_cast<const unsigned*>(hid + ((tid < R ? tid : R - 1) & ~1));
}
// Keeps the uses of a loaded value below this point: the compiler otherwise moves the conversion up into the branch
// of the load, where it waits for every load the wavefront has issued so far before the next one is issued.
__device__ __forceinline__ void use_below(unsigned& raw) { asm volatile("" : "+v"(raw)); }
// activation (0 none, 1 tanh, 2 sigmoid) into LDS; zeros from R to the end of the last round of 128
template <int ACT>
__device__ __forceinline__ void hidden_store(float* __restrict__ hs, unsigned raw, int R, int wave, int tid) {
  if (wave * 64 < ((R + 127) & ~127)) {
    float v = 0.0f;
    if (wave * 64 < R) {
      v = h2f(__builtin_bit_cast(half_t, static_cast<unsigned short>(raw >> (16 * (tid & 1)))));
      if (ACT == 1) v = tanh_f(v);
      if (ACT == 2) v = sigmoid_f(v);
      if (tid >= R) v = 0.0f;
    }
    hs[tid] = v;
  }
}

// F16: the WKV state is fp16 and the step follows the fp16-state recurrence (wkv7_f16state.h): a wavefront
// holds the head's 64 state rows of one batch row, one per lane, and does the step itself between its per-channel
// work and the GroupNorm - the other wavefronts are done after the rank-outs, two barriers in all.
//
// ROWS: batch rows of one head that a block serves (consecutive rows; the batch is a multiple of ROWS).  The head's
// LoRA rows - most of a block's bytes - are loaded once and meet the hidden vectors of every row; each row has its
// own state slice per thread, and wavefront r does the per-channel work of row r.  With B*H/ROWS blocks a batch of
// 8 or 16 rows fits the chip in one round instead of 2 or 4.
template <bool F16, int ROWS>
__global__ __launch_bounds__(kStepThreads) void tmix_step_kernel(TmixStepArgs p) {
  __shared__ __align__(16) half_t ops16[ROWS][5][kHead];  // fp16-state mode: a~, b~, k', decay delta, r
  __shared__ __align__(16) float hs[ROWS][4][kStepMaxR];  // activated LoRA hidden vectors: w, a, g, v
  __shared__ __align__(16) float lo[ROWS][4][kHead];      // rank-out results per channel: w12, a12, g, v-gate logit
  __shared__ __align__(16) float vec[ROWS][6][kHead];     // WKV operands r, d, k', a~, b~ and the mixed v
  __shared__ float yv[ROWS][kHead];                       // y of the step, rounded to fp16

  const bool split = ROWS == 1 && p.gate_out != nullptr;
  const int n_heads = (p.B / ROWS) * p.H;
  const bool gate_block = ROWS == 1 && static_cast<int>(blockIdx.x) >= n_heads;
  const int bg = gate_block ? blockIdx.x - n_heads : blockIdx.x;
  const int b0 = (bg / p.H) * ROWS;  // first batch row of the block
  const int h = bg % p.H;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int i = tid / kStepLanes;  // channel within the head / state row
  const int q = tid % kStepLanes;
  const int c = h * kHead + i;
  // the batch row whose per-channel work this wavefront does (wavefronts past ROWS do none)
  const int bw = b0 + (wave < ROWS ? wave : 0);
  const int rs = wave < ROWS ? wave : 0;
  const int64_t row = static_cast<int64_t>(bw) * p.C;

  if constexpr (ROWS == 1) {
    if (gate_block) {
      // the g rank-out of the head's 64 channels, nothing else
      LoraRow g2;
      lora_row_load(g2, p.g2 + static_cast<int64_t>(c) * p.Rg, p.Rg, q);
      unsigned hraw;
      hidden_load(hraw, p.hg + static_cast<int64_t>(b0) * p.Rg, p.Rg, wave, tid);
      __builtin_amdgcn_sched_barrier(0);
      use_below(hraw);
      hidden_store<2>(hs[0][2], hraw, p.Rg, wave, tid);
      __syncthreads();
      const float gch = lora_row_dot(g2, hs[0][2], p.Rg, q);
      if (q == 0) p.gate_out[row + c] = f2h(gch);
      return;
    }
  }

  // ---- all global loads up front
  float4_t S[ROWS];
  half_t* srow16 = nullptr;
  half2_t S16[kPairs16];
  int phase = 0;
  const int64_t state_stride = static_cast<int64_t>(p.H) * kHead * kHead;  // one batch row's states
  if constexpr (F16) {
    if (wave < ROWS) {  // state row `lane` of the head: 128 bytes
      srow16 = p.state16 + ((static_cast<int64_t>(bw) * p.H + h) * kHead + lane) * kHead;
#pragma unroll
      for (int g = 0; g < kPairs16 / 4; ++g) {
        const uint4_t t = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(srow16 + 8 * g));
#pragma unroll
        for (int e = 0; e < 4; ++e) S16[4 * g + e] = as_half2(t[e]);
      }
      phase = p.elapsed[bw];
    }
  } else {
    const float* srow = p.state + ((static_cast<int64_t>(b0) * p.H + h) * kHead + i) * kHead + 4 * q;
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
      S[r] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(srow + r * state_stride));
  }
  LoraRow w2, a2, g2, v2;
  lora_row_load(w2, p.w2 + static_cast<int64_t>(c) * p.Rw, p.Rw, q);
  lora_row_load(a2, p.a2 + static_cast<int64_t>(c) * p.Ra, p.Ra, q);
  if (!split) lora_row_load(g2, p.g2 + static_cast<int64_t>(c) * p.Rg, p.Rg, q);
  if (p.hv) lora_row_load(v2, p.v2 + static_cast<int64_t>(c) * p.Rv, p.Rv, q);
  // Activated hidden vectors and per-channel scalars: only the loads here, as raw fp16 - a conversion next to its
  // load would make the wavefront wait for everything it has requested so far before it requests the rest (loads
  // return in order), one trip to memory after another.  The scalars: wavefront r for batch row r, lane = channel.
  unsigned hw_raw[ROWS], ha_raw[ROWS], hg_raw[ROWS], hv_raw[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int64_t bi = b0 + r;
    hidden_load(hw_raw[r], p.hw + bi * p.Rw, p.Rw, wave, tid);
    hidden_load(ha_raw[r], p.ha + bi * p.Ra, p.Ra, wave, tid);
    if (!split) hidden_load(hg_raw[r], p.hg + bi * p.Rg, p.Rg, wave, tid);
    if (p.hv) hidden_load(hv_raw[r], p.hv + bi * p.Rv, p.Rv, wave, tid);
  }
  const half_t hzero = static_cast<half_t>(0.0f);
  half_t kv_h = hzero, rv_h = hzero, vv_h = hzero, kkw_h = hzero, a0_h = hzero, ka_h = hzero, w0_h = hzero, rk_h = hzero,
         lnw_h = hzero, lnb_h = hzero, v0_h = hzero, vf_h = hzero, shift_h = hzero;
  const int cl = h * kHead + lane;  // the per-channel wavefronts' channel
  if (wave < ROWS) {
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
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    use_below(hw_raw[r]);
    use_below(ha_raw[r]);
    if (!split) use_below(hg_raw[r]);
    if (p.hv) use_below(hv_raw[r]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    hidden_store<1>(hs[r][0], hw_raw[r], p.Rw, wave, tid);
    hidden_store<0>(hs[r][1], ha_raw[r], p.Ra, wave, tid);
    if (!split) hidden_store<2>(hs[r][2], hg_raw[r], p.Rg, wave, tid);
    if (p.hv) hidden_store<0>(hs[r][3], hv_raw[r], p.Rv, wave, tid);
  }
  const float kv = h2f(kv_h), rv = h2f(rv_h), vv = h2f(vv_h), kkw = h2f(kkw_h), a0 = h2f(a0_h), ka = h2f(ka_h),
              w0 = h2f(w0_h), rk = h2f(rk_h), lnw = h2f(lnw_h), lnb = h2f(lnb_h), v0 = h2f(v0_h), vf = h2f(vf_h);
  __syncthreads();

  // ---- LoRA rank-outs for channel i (fp32 sums over the 16 lanes), every row of the block (a loop that stays a
  // loop: unrolled, the rows' LDS reads are all moved to the front and spill)
#pragma nounroll
  for (int r = 0; r < ROWS; ++r) {
    const float w12 = round_h(lora_row_dot(w2, hs[r][0], p.Rw, q));
    const float a12 = round_h(lora_row_dot(a2, hs[r][1], p.Ra, q));
    const float gch = split ? 1.0f : round_h(lora_row_dot(g2, hs[r][2], p.Rg, q));
    const float vdot = p.hv ? lora_row_dot(v2, hs[r][3], p.Rv, q) : 0.0f;
    if (q == 0) {
      lo[r][0][i] = w12;
      lo[r][1][i] = a12;
      lo[r][2][i] = gch;
      lo[r][3][i] = vdot;
    }
  }
  __syncthreads();

  // ---- per channel, wavefront r for row r: v-residual gate, kk normalise over the head, a-gate, decay
  float v_use = vv, k2 = 0.0f, gch = 0.0f;
  if constexpr (F16) {
    if (wave >= ROWS) return;
  }
  if (wave < ROWS) {
    const float w12 = lo[rs][0][lane];
    const float a12 = lo[rs][1][lane];
    gch = lo[rs][2][lane];
    if (p.hv) {
      const float gate = sigmoid_f(v0 + lo[rs][3][lane]);
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
      ops16[rs][0][lane] = f2h(-kk);
      ops16[rs][1][lane] = f2h(kk * av);
      ops16[rs][2][lane] = f2h(k2);
      ops16[rs][3][lane] = decay_delta16_of(w12 + w0, phase + cl);  // (w12 + w0 unrounded: a single-token call)
      ops16[rs][4][lane] = f2h(rv);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const half_t y16 =
          wkv16_row_step(S16, ops16[rs][0], ops16[rs][1], ops16[rs][2], ops16[rs][3], ops16[rs][4], f2h(v_use));
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
    vec[rs][0][lane] = rv;
    vec[rs][1][lane] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
    vec[rs][2][lane] = k2;
    vec[rs][3][lane] = round_h(-kk);
    vec[rs][4][lane] = round_h(kk * av);
    vec[rs][5][lane] = v_use;
  }
  __syncthreads();

  // ---- WKV step on row i, this lane's 4 columns, for every batch row of the block
  if constexpr (!F16) {
    // (the state addresses are formed again, from a thread index the compiler cannot match with the one the loads
    // used: kept from the loads to here they are two registers per batch row)
    int tid2 = tid;
    asm volatile("" : "+v"(tid2));
    float* srow = p.state + ((static_cast<int64_t>(b0) * p.H + h) * kHead + tid2 / kStepLanes) * kHead +
                  4 * (tid2 % kStepLanes);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int j = 4 * q;
      float4_t s4 = S[r];
      const float vi = vec[r][5][i];
      const float4_t a4 = *reinterpret_cast<const float4_t*>(&vec[r][3][j]);
      float sa = s4.x * a4.x;
      sa = fmaf(s4.y, a4.y, sa);
      sa = fmaf(s4.z, a4.z, sa);
      sa = fmaf(s4.w, a4.w, sa);
      sa = row16_sum(sa);
      const float4_t d4 = *reinterpret_cast<const float4_t*>(&vec[r][1][j]);
      const float4_t k4 = *reinterpret_cast<const float4_t*>(&vec[r][2][j]);
      const float4_t b4 = *reinterpret_cast<const float4_t*>(&vec[r][4][j]);
      const float4_t r4 = *reinterpret_cast<const float4_t*>(&vec[r][0][j]);
      s4.x = fmaf(s4.x, d4.x, fmaf(sa, b4.x, k4.x * vi));
      s4.y = fmaf(s4.y, d4.y, fmaf(sa, b4.y, k4.y * vi));
      s4.z = fmaf(s4.z, d4.z, fmaf(sa, b4.z, k4.z * vi));
      s4.w = fmaf(s4.w, d4.w, fmaf(sa, b4.w, k4.w * vi));
      __builtin_nontemporal_store(s4, reinterpret_cast<float4_t*>(srow + r * state_stride));
      float yy = s4.x * r4.x;
      yy = fmaf(s4.y, r4.y, yy);
      yy = fmaf(s4.z, r4.z, yy);
      yy = fmaf(s4.w, r4.w, yy);
      yy = round_h(row16_sum(yy));  // the reference stores y as fp16 before the GroupNorm kernel reads it
      if (q == 0) yv[r][i] = yy;
    }
  }
  __syncthreads();

  // ---- per-head GroupNorm (two-pass), bonus term, gate: wavefront r for row r, sums inside the wavefront
  if (wave < ROWS) {
    const float yy = yv[rs][lane];
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

// Rows per block: as many (1, 2 or 4, dividing the batch) as it takes to bring the launch down to one round of
// blocks on the chip.  The fp16-state mode and the split mode keep one row per block.
int tmix_step_rows_per_block(int B, int H, bool one_row_only) {
  int rows = 1;
  if (one_row_only) return rows;
  const int cus = device_cu_count();
  while (rows < 4 && B % (rows * 2) == 0 && B * H / rows > cus) rows *= 2;
  return rows;
}

int tmix_step_launch(hipStream_t st, const TmixStepArgs& p) {
  RWKV_REQUIRE(p.B > 0 && p.H > 0 && p.C == p.H * kHead, "tmix_step: bad shape");
  RWKV_REQUIRE(p.Rw % 8 == 0 && p.Ra % 8 == 0 && p.Rg % 8 == 0 && p.Rv % 8 == 0 && p.Rw <= kStepMaxR &&
                   p.Ra <= kStepMaxR && p.Rg <= kStepMaxR && p.Rv <= kStepMaxR,
               "tmix_step: LoRA ranks must be multiples of 8, at most %d", kStepMaxR);
  RWKV_REQUIRE((p.gate_out == nullptr) == (p.y2_pre == nullptr), "tmix_step: split mode needs both y2_pre and gate_out");
  RWKV_REQUIRE((p.state != nullptr) != (p.state16 != nullptr), "tmix_step: exactly one of the fp32 and the fp16 state");
  RWKV_REQUIRE(p.state16 == nullptr || p.elapsed != nullptr, "tmix_step: the fp16 state needs the elapsed counters");
  const int rpb = p.rows_per_block > 0 ? p.rows_per_block
                                       : tmix_step_rows_per_block(p.B, p.H, p.gate_out != nullptr || p.state16 != nullptr);
  RWKV_REQUIRE(rpb == 1 || rpb == 2 || rpb == 4, "tmix_step: 1, 2 or 4 rows per block");
  RWKV_REQUIRE(p.B % rpb == 0, "tmix_step: the batch must be a multiple of the rows per block");
  RWKV_REQUIRE(rpb == 1 || (p.gate_out == nullptr && p.state16 == nullptr),
               "tmix_step: split mode and the fp16 state take one row per block");
  const int blocks = p.B / rpb * p.H * (p.gate_out ? 2 : 1);
  if (p.state16) {
    hipLaunchKernelGGL((tmix_step_kernel<true, 1>), dim3(blocks), dim3(kStepThreads), 0, st, p);
  } else if (rpb == 4) {
    hipLaunchKernelGGL((tmix_step_kernel<false, 4>), dim3(blocks), dim3(kStepThreads), 0, st, p);
  } else if (rpb == 2) {
    hipLaunchKernelGGL((tmix_step_kernel<false, 2>), dim3(blocks), dim3(kStepThreads), 0, st, p);
  } else {
    hipLaunchKernelGGL((tmix_step_kernel<false, 1>), dim3(blocks), dim3(kStepThreads), 0, st, p);
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv
