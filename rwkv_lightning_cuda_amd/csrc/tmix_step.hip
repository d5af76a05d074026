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
// Layout: 256 threads = 64 channels x 4 lanes.  Lane q of channel i owns a quarter of that channel's LoRA
// rows (8-element chunks q, q+4, ...) and, for the state, row i's columns {16p + 4q .. +3 : p = 0..3} so
// that the four lanes of a row read 64 contiguous bytes per load.  Row sums finish with a 4-lane
// butterfly (two DPP/shuffle steps).
#include "ops.h"

namespace rwkv {

constexpr int kStepMaxR = 512;

__device__ __forceinline__ float quad_sum(float v) {
  v += __shfl_xor(v, 1, 64);
  v += __shfl_xor(v, 2, 64);
  return v;
}

// partial dot of this lane's chunks of one LoRA row against the activated hidden vector in LDS
__device__ __forceinline__ float lora_row_partial(const half_t* __restrict__ wrow, const float* __restrict__ hs, int R,
                                                  int q) {
  float acc = 0.0f;
  for (int r0 = q * 8; r0 < R; r0 += 32) {
    const half8_t w = *reinterpret_cast<const half8_t*>(wrow + r0);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = fmaf(hs[r0 + e], h2f(w[e]), acc);
  }
  return acc;
}

__global__ __launch_bounds__(256) void tmix_step_kernel(TmixStepArgs p) {
  __shared__ __align__(16) float hs[4][kStepMaxR];  // activated LoRA hidden vectors: w, a, g, v
  __shared__ __align__(16) float vec[6][kHead];     // r, d, k', a~, b~ (WKV operands) and y
  __shared__ float red[3][4];

  const int bh = blockIdx.x;
  const int bi = bh / p.H;
  const int h = bh - bi * p.H;
  const int tid = threadIdx.x;
  const int i = tid >> 2;  // channel within the head / state row
  const int q = tid & 3;
  const int c = h * kHead + i;
  const int64_t row = static_cast<int64_t>(bi) * p.C;

  // state row slices first: the longest-latency loads
  float* srow = p.state + (static_cast<int64_t>(bh) * kHead + i) * kHead;
  float4_t S[4];
#pragma unroll
  for (int pp = 0; pp < 4; ++pp) S[pp] = *reinterpret_cast<const float4_t*>(srow + 16 * pp + 4 * q);

  // activated hidden vectors into LDS
  const int ranks[4] = {p.Rw, p.Ra, p.Rg, p.Rv};
  const half_t* hid[4] = {p.hw + static_cast<int64_t>(bi) * p.Rw, p.ha + static_cast<int64_t>(bi) * p.Ra,
                          p.hg + static_cast<int64_t>(bi) * p.Rg, p.hv ? p.hv + static_cast<int64_t>(bi) * p.Rv : nullptr};
#pragma unroll
  for (int gidx = 0; gidx < 4; ++gidx) {
    if (hid[gidx] == nullptr) continue;
    for (int r = tid; r < ranks[gidx]; r += 256) {
      float hv = h2f(hid[gidx][r]);
      if (gidx == 0) hv = tanhf(hv);
      if (gidx == 2) hv = sigmoid_f(hv);
      hs[gidx][r] = hv;
    }
  }
  const float kv = h2f(p.k[row + c]);
  const float rv = h2f(p.r[row + c]);
  const float vv = h2f(p.v[row + c]);
  __syncthreads();

  // LoRA rank-outs for channel c (fp32 sums, completed across the 4 lanes)
  const float w_sum = quad_sum(lora_row_partial(p.w2 + static_cast<int64_t>(c) * p.Rw, hs[0], p.Rw, q));
  const float a_sum = quad_sum(lora_row_partial(p.a2 + static_cast<int64_t>(c) * p.Ra, hs[1], p.Ra, q));
  const float g_sum = quad_sum(lora_row_partial(p.g2 + static_cast<int64_t>(c) * p.Rg, hs[2], p.Rg, q));
  float v_use = vv;
  if (p.hv) {
    const float v_sum = quad_sum(lora_row_partial(p.v2 + static_cast<int64_t>(c) * p.Rv, hs[3], p.Rv, q));
    const float gate = sigmoid_f(h2f(p.v0[c]) + v_sum);
    v_use = round_h(vv + (h2f(p.v_first[row + c]) - vv) * gate);
  } else if (p.v_first_out && q == 0) {
    p.v_first_out[row + c] = f2h(vv);  // layer 0: v_first = v
  }
  const float w12 = round_h(w_sum);
  const float a12 = round_h(a_sum);
  const float gch = round_h(g_sum);

  // kk normalise over the head (each channel counted once: lane q == 0)
  const float u = kv * h2f(p.k_k[c]);
  float part = (q == 0) ? u * u : 0.0f;
  part = wave_sum(part);
  if ((tid & 63) == 0) red[0][tid >> 6] = part;
  __syncthreads();
  const float total = red[0][0] + red[0][1] + red[0][2] + red[0][3];
  const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
  const float kk = u * inv;
  const float av = sigmoid_f(h2f(p.a0[c]) + a12);
  const float ka = h2f(p.k_a[c]);
  const float k2 = round_h(kv * fmaf(av, ka, 1.0f - ka));
  if (q == 0) {
    const float wraw = round_h(w12 + h2f(p.w0[c]));
    vec[0][i] = rv;
    vec[1][i] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
    vec[2][i] = k2;
    vec[3][i] = round_h(-kk);
    vec[4][i] = round_h(kk * av);
  }
  __syncthreads();

  // WKV step on row i, this lane's 16 columns
  float sa = 0.0f;
#pragma unroll
  for (int pp = 0; pp < 4; ++pp) {
    const float4_t a4 = *reinterpret_cast<const float4_t*>(&vec[3][16 * pp + 4 * q]);
    sa = fmaf(S[pp].x, a4.x, sa);
    sa = fmaf(S[pp].y, a4.y, sa);
    sa = fmaf(S[pp].z, a4.z, sa);
    sa = fmaf(S[pp].w, a4.w, sa);
  }
  sa = quad_sum(sa);
  float yy = 0.0f;
#pragma unroll
  for (int pp = 0; pp < 4; ++pp) {
    const int j = 16 * pp + 4 * q;
    const float4_t d4 = *reinterpret_cast<const float4_t*>(&vec[1][j]);
    const float4_t k4 = *reinterpret_cast<const float4_t*>(&vec[2][j]);
    const float4_t b4 = *reinterpret_cast<const float4_t*>(&vec[4][j]);
    const float4_t r4 = *reinterpret_cast<const float4_t*>(&vec[0][j]);
    float4_t s = S[pp];
    s.x = fmaf(s.x, d4.x, fmaf(sa, b4.x, k4.x * v_use));
    s.y = fmaf(s.y, d4.y, fmaf(sa, b4.y, k4.y * v_use));
    s.z = fmaf(s.z, d4.z, fmaf(sa, b4.z, k4.z * v_use));
    s.w = fmaf(s.w, d4.w, fmaf(sa, b4.w, k4.w * v_use));
    yy = fmaf(s.x, r4.x, yy);
    yy = fmaf(s.y, r4.y, yy);
    yy = fmaf(s.z, r4.z, yy);
    yy = fmaf(s.w, r4.w, yy);
    *reinterpret_cast<float4_t*>(srow + j) = s;
  }
  yy = round_h(quad_sum(yy));  // the reference stores y as fp16 before the GroupNorm kernel reads it

  // per-head GroupNorm (two-pass), bonus term, gate
  float s1 = (q == 0) ? yy : 0.0f;
  float s3 = (q == 0) ? rv * k2 * h2f(p.r_k[c]) : 0.0f;
  s1 = wave_sum(s1);
  s3 = wave_sum(s3);
  if ((tid & 63) == 0) {
    red[1][tid >> 6] = s1;
    red[2][tid >> 6] = s3;
  }
  __syncthreads();
  const float mean = (red[1][0] + red[1][1] + red[1][2] + red[1][3]) * (1.0f / 64.0f);
  const float rkv = red[2][0] + red[2][1] + red[2][2] + red[2][3];
  const float dlt = yy - mean;
  float s2 = (q == 0) ? dlt * dlt : 0.0f;
  s2 = wave_sum(s2);
  __syncthreads();  // red[0] reuse
  if ((tid & 63) == 0) red[0][tid >> 6] = s2;
  __syncthreads();
  const float var = (red[0][0] + red[0][1] + red[0][2] + red[0][3]) * (1.0f / 64.0f);
  const float rstd = rsqrtf(var + kLnxEps);
  if (q == 0) {
    const float o = (dlt * rstd * h2f(p.lnx_w[c]) + h2f(p.lnx_b[c]) + rkv * v_use) * gch;
    p.y2[row + c] = f2h(o);
  }
}

int tmix_step_launch(hipStream_t st, const TmixStepArgs& p) {
  RWKV_REQUIRE(p.B > 0 && p.H > 0 && p.C == p.H * kHead, "tmix_step: bad shape");
  RWKV_REQUIRE(p.Rw % 8 == 0 && p.Ra % 8 == 0 && p.Rg % 8 == 0 && p.Rv % 8 == 0 && p.Rw <= kStepMaxR &&
                   p.Ra <= kStepMaxR && p.Rg <= kStepMaxR && p.Rv <= kStepMaxR,
               "tmix_step: LoRA ranks must be multiples of 8, at most %d", kStepMaxR);
  hipLaunchKernelGGL(tmix_step_kernel, dim3(p.B * p.H), dim3(256), 0, st, p);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv
