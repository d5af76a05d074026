// W8A16 / W4A16 weight formats: quantise-on-load and dequantise kernels.
//
// The reference keeps fp16 weights only (cuda/rwkv7_v3a_ops.cu:464-560 reads `half` rows), so these
// formats have no upstream counterpart.  The arithmetic below is ordered so that a scalar CPU
// implementation using IEEE fp32 division, rint (ties-to-even) and fp16 RNE gives the same bits:
//   W8 (per output row):  amax = max|w|;  s = f16(amax / 127);  q = clamp(rint(w / f32(s)), -127, 127)
//                         (s == 0 -> q = 0);  dequant = f16(f32(s) * q)
//   W4 (per 128 along K): lo = min(min w, 0), hi = max(max w, 0);  s = f16((hi - lo) / 15) (0 -> 1);
//                         zp = clamp(rint(-lo / f32(s)), 0, 15);  q = clamp(rint(w / f32(s)) + zp, 0, 15)
//                         dequant = f16(f32(s) * (q - zp));  two codes per byte, even k in the low nibble
#include "common.h"

namespace rwkv {

__global__ __launch_bounds__(256) void quantize_w8_kernel(int K, const half_t* __restrict__ w,
                                                          int8_t* __restrict__ q, half_t* __restrict__ scale) {
  __shared__ float red[4];
  const int64_t n = blockIdx.x;
  const half_t* row = w + n * K;
  float amax = 0.0f;
  for (int k = threadIdx.x; k < K; k += 256) amax = fmaxf(amax, fabsf(h2f(row[k])));
  amax = wave_max(amax);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const half_t sh = f2h(amax / 127.0f);
  const float s = h2f(sh);
  if (threadIdx.x == 0) scale[n] = sh;
  for (int k = threadIdx.x; k < K; k += 256) {
    float v = 0.0f;
    if (s > 0.0f) v = rintf(h2f(row[k]) / s);
    v = fminf(127.0f, fmaxf(-127.0f, v));
    q[n * K + k] = static_cast<int8_t>(v);
  }
}

__global__ __launch_bounds__(256) void dequant_w8_kernel(int64_t total, int K, const int8_t* __restrict__ q,
                                                         const half_t* __restrict__ scale, half_t* __restrict__ w) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  w[i] = f2h(h2f(scale[i / K]) * static_cast<float>(q[i]));
}

// one wave per 128-wide group, two elements per lane
__global__ __launch_bounds__(256) void quantize_w4_kernel(int64_t groups, const half_t* __restrict__ w,
                                                          uint8_t* __restrict__ q, half_t* __restrict__ scale,
                                                          uint8_t* __restrict__ zp) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (g >= groups) return;
  const int lane = threadIdx.x & 63;
  const float v0 = h2f(w[g * 128 + lane * 2]);
  const float v1 = h2f(w[g * 128 + lane * 2 + 1]);
  float lo = fminf(fminf(v0, v1), 0.0f);
  float hi = fmaxf(fmaxf(v0, v1), 0.0f);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    lo = fminf(lo, __shfl_xor(lo, off, 64));
    hi = fmaxf(hi, __shfl_xor(hi, off, 64));
  }
  half_t sh = f2h((hi - lo) / 15.0f);
  if (h2f(sh) == 0.0f) sh = f2h(1.0f);
  const float s = h2f(sh);
  const float z = fminf(15.0f, fmaxf(0.0f, rintf(-lo / s)));
  const float c0 = fminf(15.0f, fmaxf(0.0f, rintf(v0 / s) + z));
  const float c1 = fminf(15.0f, fmaxf(0.0f, rintf(v1 / s) + z));
  q[g * 64 + lane] = static_cast<uint8_t>(static_cast<uint32_t>(c0) | (static_cast<uint32_t>(c1) << 4));
  if (lane == 0) {
    scale[g] = sh;
    zp[g] = static_cast<uint8_t>(z);
  }
}

__global__ __launch_bounds__(256) void dequant_w4_kernel(int64_t total, const uint8_t* __restrict__ q,
                                                         const half_t* __restrict__ scale,
                                                         const uint8_t* __restrict__ zp, half_t* __restrict__ w) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // element index
  if (i >= total) return;
  const int64_t g = i >> 7;
  const uint8_t byte = q[i >> 1];
  const int code = (i & 1) ? (byte >> 4) : (byte & 15);
  w[i] = f2h(h2f(scale[g]) * static_cast<float>(code - static_cast<int>(zp[g])));
}

// Synthetic weights for benchmarks: value i is mean + std * N(0,1) drawn from a counter-based hash of
// (seed, i) through Box-Muller, rounded to fp16.
__global__ __launch_bounds__(256) void fill_normal_f16_kernel(int64_t n, uint64_t seed, float mean, float stdv,
                                                              half_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * static_cast<uint64_t>(i + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  const float u1 = (static_cast<float>(z >> 40) + 1.0f) * (1.0f / 16777216.0f);       // (0,1]
  const float u2 = static_cast<float>((z >> 16) & 0xffffffu) * (1.0f / 16777216.0f);  // [0,1)
  const float g = sqrtf(-2.0f * __logf(u1)) * __cosf(6.283185307179586f * u2);
  out[i] = f2h(mean + stdv * g);
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_fill_normal_f16(rwkv_stream_t s, int64_t n, uint64_t seed, float mean, float stdv, void* out) {
  RWKV_REQUIRE(n > 0 && out, "fill_normal_f16: bad arguments");
  hipLaunchKernelGGL(fill_normal_f16_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, as_stream(s), n, seed, mean, stdv,
                     static_cast<half_t*>(out));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_quantize_w8(rwkv_stream_t s, int N, int K, const void* w_f16, void* q, void* scale) {
  RWKV_REQUIRE(N > 0 && K > 0 && w_f16 && q && scale, "quantize_w8: bad arguments");
  hipLaunchKernelGGL(quantize_w8_kernel, dim3(N), dim3(256), 0, as_stream(s), K, static_cast<const half_t*>(w_f16),
                     static_cast<int8_t*>(q), static_cast<half_t*>(scale));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_dequant_w8(rwkv_stream_t s, int N, int K, const void* q, const void* scale, void* w_f16) {
  RWKV_REQUIRE(N > 0 && K > 0 && w_f16 && q && scale, "dequant_w8: bad arguments");
  const int64_t total = static_cast<int64_t>(N) * K;
  hipLaunchKernelGGL(dequant_w8_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, as_stream(s), total, K,
                     static_cast<const int8_t*>(q), static_cast<const half_t*>(scale), static_cast<half_t*>(w_f16));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_quantize_w4(rwkv_stream_t s, int N, int K, const void* w_f16, void* q, void* scale, void* zp) {
  RWKV_REQUIRE(N > 0 && K > 0 && K % 128 == 0 && w_f16 && q && scale && zp,
               "quantize_w4: K (%d) must be a positive multiple of 128", K);
  const int64_t groups = static_cast<int64_t>(N) * (K / 128);
  hipLaunchKernelGGL(quantize_w4_kernel, dim3(ceil_div(groups, 4)), dim3(256), 0, as_stream(s), groups,
                     static_cast<const half_t*>(w_f16), static_cast<uint8_t*>(q), static_cast<half_t*>(scale),
                     static_cast<uint8_t*>(zp));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_dequant_w4(rwkv_stream_t s, int N, int K, const void* q, const void* scale, const void* zp,
                        void* w_f16) {
  RWKV_REQUIRE(N > 0 && K > 0 && K % 128 == 0 && w_f16 && q && scale && zp,
               "dequant_w4: K (%d) must be a positive multiple of 128", K);
  const int64_t total = static_cast<int64_t>(N) * K;
  hipLaunchKernelGGL(dequant_w4_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, as_stream(s), total,
                     static_cast<const uint8_t*>(q), static_cast<const half_t*>(scale),
                     static_cast<const uint8_t*>(zp), static_cast<half_t*>(w_f16));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // extern "C"
