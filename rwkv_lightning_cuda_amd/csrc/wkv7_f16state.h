// Pieces of the fp16-state WKV7 recurrence shared by its sequence kernel (wkv7_f16state.hip) and the single-launch
// decode time-mix core (tmix_step.hip): the same functions, so both produce the same bits.
// Reference: cuda/rwkv7_wkv_fp16_v2.cu:41-52 (decay delta with dither), :157-193 (one token).
#pragma once

#include "ops.h"

namespace rwkv {

constexpr int kPairs16 = kHead / 2;  // half2 pairs per state row

__device__ __forceinline__ half2_t pk_fma16(half2_t x, half2_t y, half2_t z) { return __builtin_elementwise_fma(x, y, z); }

// f16(exp2f(-e^-1/2 log2e / (1 + exp2f(-log2e * w))) - 1 + dither(phase));
// dither(x) = 2^-41 * float(int32(2654435769 * x))
__device__ __forceinline__ half_t decay_delta16_of(float w, int phase) {
  const unsigned prod = 2654435769u * static_cast<unsigned>(phase);
  const float dither = 4.547473508864641e-13f * static_cast<float>(static_cast<int>(prod));
  const float d = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * w))) - 1.0f + dither;
  return f2h(d);
}
// w = w_raw (+ w0[c], unrounded, as the reference's _w0 launchers)
__device__ __forceinline__ half_t decay_delta16(half_t w_raw, const half_t* __restrict__ w0, int c, int phase) {
  float w = h2f(w_raw);
  if (w0) w += h2f(w0[c]);
  return decay_delta16_of(w, phase);
}

__device__ __forceinline__ void read_pairs16(const half_t* __restrict__ src, half2_t (&dst)[kPairs16]) {
#pragma unroll
  for (int q = 0; q < kPairs16 / 4; ++q) {
    const uint4_t t = *reinterpret_cast<const uint4_t*>(src + 8 * q);
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[4 * q + e] = as_half2(t[e]);
  }
}

// One token for state row S (this lane's row) given the per-column operands in (shared) memory and the row's v;
// returns y of the row.  The two chains run over the pairs in order: fp16 sums do not associate.
__device__ __forceinline__ half_t wkv16_row_step(half2_t (&S)[kPairs16], const half_t* __restrict__ a, const half_t* __restrict__ b,
                                                 const half_t* __restrict__ k, const half_t* __restrict__ wd,
                                                 const half_t* __restrict__ r, half_t v_cur) {
  half2_t vec[kPairs16];
  read_pairs16(a, vec);
  half2_t sa2 = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
#pragma unroll
  for (int j = 0; j < kPairs16; ++j) sa2 = pk_fma16(vec[j], S[j], sa2);
  const half_t sa = sa2[0] + sa2[1];
  const half2_t sa_b = {sa, sa};
  const half2_t vv = {v_cur, v_cur};
  half2_t bv[kPairs16], kv[kPairs16], wv[kPairs16];
  read_pairs16(b, bv);
  read_pairs16(k, kv);
  read_pairs16(wd, wv);
  read_pairs16(r, vec);
  half2_t y2 = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
#pragma unroll
  for (int j = 0; j < kPairs16; ++j) {
    const half2_t s = S[j];
    const half2_t s_new = pk_fma16(s, wv[j], pk_fma16(kv[j], vv, pk_fma16(sa_b, bv[j], s)));
    S[j] = s_new;
    y2 = pk_fma16(s_new, vec[j], y2);
  }
  return y2[0] + y2[1];
}

}  // namespace rwkv
