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
// LoRA rows.  Row sums finish with a 16-lane butterfly.
#include "ops.h"

namespace rwkv {

constexpr int kStepMaxR = 512;
constexpr int kStepLanes = 16;                       // lanes per channel
constexpr int kStepThreads = kHead * kStepLanes;     // 1024
constexpr int kStepWaves = kStepThreads / 64;        // 16
constexpr int kStepChunks = kStepMaxR / (8 * kStepLanes);  // 4

struct LoraRow {
  half8_t w[kStepChunks];
};

__device__ __forceinline__ LoraRow lora_row_load(const half_t* __restrict__ wrow, int R, int q) {
  LoraRow row;
#pragma unroll
  for (int ii = 0; ii < kStepChunks; ++ii) {
    const int r0 = (q + kStepLanes * ii) * 8;
    if (r0 < R) {
      row.w[ii] = *reinterpret_cast<const half8_t*>(wrow + r0);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) row.w[ii][e] = static_cast<half_t>(0.0f);
    }
  }
  return row;
}

__device__ __forceinline__ float lora_row_dot(const LoraRow& row, const float* __restrict__ hs, int R, int q) {
  float acc = 0.0f;
#pragma unroll
  for (int ii = 0; ii < kStepChunks; ++ii) {
    const int r0 = (q + kStepLanes * ii) * 8;
    if (r0 < R) {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = fmaf(hs[r0 + e], h2f(row.w[ii][e]), acc);
    }
  }
  return group_sum<kStepLanes>(acc);
}

// sum over the block of a value that is non-zero in one lane per channel; every thread gets the result
__device__ __forceinline__ float head_sum(float v, float* scratch) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < kStepWaves; ++w) t += scratch[w];
  return t;
}

__global__ __launch_bounds__(kStepThreads) void tmix_step_kernel(TmixStepArgs p) {
  __shared__ __align__(16) float hs[4][kStepMaxR];  // activated LoRA hidden vectors: w, a, g, v
  __shared__ __align__(16) float vec[5][kHead];     // WKV operands r, d, k', a~, b~
  __shared__ float red[4][kStepWaves];

  const int bh = blockIdx.x;
  const int bi = bh / p.H;
  const int h = bh - bi * p.H;
  const int tid = threadIdx.x;
  const int i = tid / kStepLanes;  // channel within the head / state row
  const int q = tid % kStepLanes;
  const int c = h * kHead + i;
  const int64_t row = static_cast<int64_t>(bi) * p.C;

  // the LN output that the r/k/v launch computed in its prologue becomes the shift row of the state (that
  // launch could not store it itself: other blocks of it were still reading the old row)
  if (p.shift_dst && tid < kHead) {
    const int64_t o = row + h * kHead + tid;
    p.shift_dst[o] = p.shift_src[o];
  }

  // ---- all global loads up front
  float* srow = p.state + (static_cast<int64_t>(bh) * kHead + i) * kHead + 4 * q;
  float4_t S = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(srow));
  const LoraRow w2 = lora_row_load(p.w2 + static_cast<int64_t>(c) * p.Rw, p.Rw, q);
  const LoraRow a2 = lora_row_load(p.a2 + static_cast<int64_t>(c) * p.Ra, p.Ra, q);
  const LoraRow g2 = lora_row_load(p.g2 + static_cast<int64_t>(c) * p.Rg, p.Rg, q);
  LoraRow v2 = {};
  if (p.hv) v2 = lora_row_load(p.v2 + static_cast<int64_t>(c) * p.Rv, p.Rv, q);
  const float kv = h2f(p.k[row + c]);
  const float rv = h2f(p.r[row + c]);
  const float vv = h2f(p.v[row + c]);
  const float kkw = h2f(p.k_k[c]);
  const float a0 = h2f(p.a0[c]);
  const float ka = h2f(p.k_a[c]);
  const float w0 = h2f(p.w0[c]);
  const float rk = h2f(p.r_k[c]);
  const float lnw = h2f(p.lnx_w[c]);
  const float lnb = h2f(p.lnx_b[c]);
  const float v0 = p.hv ? h2f(p.v0[c]) : 0.0f;
  const float vf = p.hv ? h2f(p.v_first[row + c]) : 0.0f;

  // activated hidden vectors into LDS
  const int ranks[4] = {p.Rw, p.Ra, p.Rg, p.Rv};
  const half_t* hid[4] = {p.hw + static_cast<int64_t>(bi) * p.Rw, p.ha + static_cast<int64_t>(bi) * p.Ra,
                          p.hg + static_cast<int64_t>(bi) * p.Rg, p.hv ? p.hv + static_cast<int64_t>(bi) * p.Rv : nullptr};
#pragma unroll
  for (int gidx = 0; gidx < 4; ++gidx) {
    if (hid[gidx] == nullptr) continue;
    for (int r = tid; r < ranks[gidx]; r += kStepThreads) {
      float hv = h2f(hid[gidx][r]);
      if (gidx == 0) hv = tanh_f(hv);
      if (gidx == 2) hv = sigmoid_f(hv);
      hs[gidx][r] = hv;
    }
  }
  __syncthreads();

  // ---- LoRA rank-outs for channel c (fp32 sums over the 16 lanes)
  const float w12 = round_h(lora_row_dot(w2, hs[0], p.Rw, q));
  const float a12 = round_h(lora_row_dot(a2, hs[1], p.Ra, q));
  const float gch = round_h(lora_row_dot(g2, hs[2], p.Rg, q));
  float v_use = vv;
  if (p.hv) {
    const float gate = sigmoid_f(v0 + lora_row_dot(v2, hs[3], p.Rv, q));
    v_use = round_h(vv + (vf - vv) * gate);
  } else if (p.v_first_out && q == 0) {
    p.v_first_out[row + c] = f2h(vv);  // layer 0: v_first = v
  }

  // ---- kk normalise over the head (each channel counted once: lane q == 0), a-gate, decay
  const float u = kv * kkw;
  const float total = head_sum((q == 0) ? u * u : 0.0f, red[0]);
  const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
  const float kk = u * inv;
  const float av = sigmoid_f(a0 + a12);
  const float k2 = round_h(kv * fmaf(av, ka, 1.0f - ka));
  if (q == 0) {
    const float wraw = round_h(w12 + w0);
    vec[0][i] = rv;
    vec[1][i] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
    vec[2][i] = k2;
    vec[3][i] = round_h(-kk);
    vec[4][i] = round_h(kk * av);
  }
  __syncthreads();

  // ---- WKV step on row i, this lane's 4 columns
  const int j = 4 * q;
  const float4_t a4 = *reinterpret_cast<const float4_t*>(&vec[3][j]);
  float sa = S.x * a4.x;
  sa = fmaf(S.y, a4.y, sa);
  sa = fmaf(S.z, a4.z, sa);
  sa = fmaf(S.w, a4.w, sa);
  sa = group_sum<kStepLanes>(sa);
  const float4_t d4 = *reinterpret_cast<const float4_t*>(&vec[1][j]);
  const float4_t k4 = *reinterpret_cast<const float4_t*>(&vec[2][j]);
  const float4_t b4 = *reinterpret_cast<const float4_t*>(&vec[4][j]);
  const float4_t r4 = *reinterpret_cast<const float4_t*>(&vec[0][j]);
  S.x = fmaf(S.x, d4.x, fmaf(sa, b4.x, k4.x * v_use));
  S.y = fmaf(S.y, d4.y, fmaf(sa, b4.y, k4.y * v_use));
  S.z = fmaf(S.z, d4.z, fmaf(sa, b4.z, k4.z * v_use));
  S.w = fmaf(S.w, d4.w, fmaf(sa, b4.w, k4.w * v_use));
  __builtin_nontemporal_store(S, reinterpret_cast<float4_t*>(srow));
  float yy = S.x * r4.x;
  yy = fmaf(S.y, r4.y, yy);
  yy = fmaf(S.z, r4.z, yy);
  yy = fmaf(S.w, r4.w, yy);
  yy = round_h(group_sum<kStepLanes>(yy));  // the reference stores y as fp16 before the GroupNorm kernel reads it

  // ---- per-head GroupNorm (two-pass), bonus term, gate
  const float mean = head_sum((q == 0) ? yy : 0.0f, red[1]) * (1.0f / 64.0f);
  const float rkv = head_sum((q == 0) ? rv * k2 * rk : 0.0f, red[2]);
  const float dlt = yy - mean;
  const float var = head_sum((q == 0) ? dlt * dlt : 0.0f, red[3]) * (1.0f / 64.0f);
  const float rstd = rsqrtf(var + kLnxEps);
  if (q == 0) {
    const float o = (dlt * rstd * lnw + lnb + rkv * v_use) * gch;
    p.y2[row + c] = f2h(o);
  }
}

int tmix_step_launch(hipStream_t st, const TmixStepArgs& p) {
  RWKV_REQUIRE(p.B > 0 && p.H > 0 && p.C == p.H * kHead, "tmix_step: bad shape");
  RWKV_REQUIRE(p.Rw % 8 == 0 && p.Ra % 8 == 0 && p.Rg % 8 == 0 && p.Rv % 8 == 0 && p.Rw <= kStepMaxR &&
                   p.Ra <= kStepMaxR && p.Rg <= kStepMaxR && p.Rv <= kStepMaxR,
               "tmix_step: LoRA ranks must be multiples of 8, at most %d", kStepMaxR);
  hipLaunchKernelGGL(tmix_step_kernel, dim3(p.B * p.H), dim3(kStepThreads), 0, st, p);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv
