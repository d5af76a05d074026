// Load-time conversions of checkpoint tensors (bf16 in the file, fp16 on the device).
//
// Reference launchers restated here (cuda/rwkv7_fast_v4_kernels.cuh:8-29, kernels cuda/rwkv7_v3a_ops.cu:70-185):
//   rwkv7_v4_bf16_to_f16_launch ............ element-wise, fp32 widening then round-to-nearest-even
//   rwkv7_v4_bf16_to_f16_transpose_launch .. the same into the transposed layout (LoRA matrices)
//   rwkv7_v4_emb_ln0_bf16_to_f16_launch .... LayerNorm(ln0) of every embedding row: two-pass fp32 statistics over the
//                                            widened bf16 row, y = f16((x - mean) * rstd * w + b) with bf16 w, b
// All three are bound by HBM and run once per model; they are written for coalescing, not tuned further.
#include "ops.h"

namespace rwkv {

__device__ __forceinline__ float bf16_to_f32(uint16_t bits) { return __uint_as_float(static_cast<uint32_t>(bits) << 16); }

// 8 elements per thread, 16-byte loads and stores; the tail element-wise
__global__ __launch_bounds__(256) void bf16_to_f16_kernel(int64_t n, const uint16_t* __restrict__ src, half_t* __restrict__ dst) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  if (i + 8 <= n) {
    const uint4_t v = *reinterpret_cast<const uint4_t*>(src + i);
    half8_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[2 * e] = f2h(bf16_to_f32(static_cast<uint16_t>(v[e] & 0xffffu)));
      o[2 * e + 1] = f2h(bf16_to_f32(static_cast<uint16_t>(v[e] >> 16)));
    }
    *reinterpret_cast<half8_t*>(dst + i) = o;
  } else {
    for (int64_t k = i; k < n; ++k) dst[k] = f2h(bf16_to_f32(src[k]));
  }
}

// src [rows, cols] -> dst [cols, rows] through a 32 x 33 LDS tile: both sides coalesced
__global__ __launch_bounds__(256) void bf16_to_f16_transpose_kernel(int rows, int cols, const uint16_t* __restrict__ src,
                                                                  half_t* __restrict__ dst) {
  __shared__ half_t tile[32][33];
  const int tx = threadIdx.x & 31;
  const int ty = threadIdx.x >> 5;  // 0..7
  const int c0 = blockIdx.x * 32;
  const int r0 = blockIdx.y * 32;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int r = r0 + ty + 8 * k;
    const int c = c0 + tx;
    if (r < rows && c < cols) tile[ty + 8 * k][tx] = f2h(bf16_to_f32(src[static_cast<int64_t>(r) * cols + c]));
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int c = c0 + ty + 8 * k;
    const int r = r0 + tx;
    if (r < rows && c < cols) dst[static_cast<int64_t>(c) * rows + r] = tile[tx][ty + 8 * k];
  }
}

// one block per embedding row
__global__ __launch_bounds__(256) void emb_ln0_kernel(int C, const uint16_t* __restrict__ emb, const uint16_t* __restrict__ w,
                                                    const uint16_t* __restrict__ b, float eps, half_t* __restrict__ out) {
  __shared__ float red[4];
  const uint16_t* row = emb + static_cast<int64_t>(blockIdx.x) * C;
  float sum = 0.0f;
  for (int c = threadIdx.x; c < C; c += 256) sum += bf16_to_f32(row[c]);
  const float mean = block_sum<4>(sum, red) / static_cast<float>(C);
  float sq = 0.0f;
  for (int c = threadIdx.x; c < C; c += 256) {
    const float d = bf16_to_f32(row[c]) - mean;
    sq = fmaf(d, d, sq);
  }
  const float rstd = rsqrtf(block_sum<4>(sq, red) / static_cast<float>(C) + eps);
  half_t* y = out + static_cast<int64_t>(blockIdx.x) * C;
  for (int c = threadIdx.x; c < C; c += 256) {
    y[c] = f2h(fmaf((bf16_to_f32(row[c]) - mean) * rstd, bf16_to_f32(w[c]), bf16_to_f32(b[c])));
  }
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_bf16_to_f16(rwkv_stream_t s, int64_t n, const void* src_bf16, void* dst_f16) {
  RWKV_REQUIRE(n >= 0 && (n == 0 || (src_bf16 && dst_f16)), "bf16_to_f16: bad arguments");
  if (n == 0) return RWKV_OK;
  RWKV_REQUIRE((reinterpret_cast<uintptr_t>(src_bf16) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst_f16) & 15) == 0,
               "bf16_to_f16: tensors must be 16-byte aligned");
  const int64_t blocks = (n + 2047) / 2048;
  RWKV_REQUIRE(blocks <= 0x7fffffff, "bf16_to_f16: %lld elements are too many for one launch", static_cast<long long>(n));
  hipLaunchKernelGGL(bf16_to_f16_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, as_stream(s), n,
                     static_cast<const uint16_t*>(src_bf16), static_cast<half_t*>(dst_f16));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_bf16_to_f16_transpose(rwkv_stream_t s, int rows, int cols, const void* src_bf16, void* dst_f16) {
  RWKV_REQUIRE(rows > 0 && cols > 0 && src_bf16 && dst_f16 && src_bf16 != dst_f16, "bf16_to_f16_transpose: bad arguments");
  hipLaunchKernelGGL(bf16_to_f16_transpose_kernel, dim3((cols + 31) / 32, (rows + 31) / 32), dim3(256), 0, as_stream(s), rows,
                     cols, static_cast<const uint16_t*>(src_bf16), static_cast<half_t*>(dst_f16));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_emb_ln0_bf16_to_f16(rwkv_stream_t s, int V, int C, const void* emb_bf16, const void* weight_bf16,
                                 const void* bias_bf16, float eps, void* out_f16) {
  RWKV_REQUIRE(V > 0 && C > 0 && emb_bf16 && weight_bf16 && bias_bf16 && out_f16, "emb_ln0: bad arguments");
  hipLaunchKernelGGL(emb_ln0_kernel, dim3(V), dim3(256), 0, as_stream(s), C, static_cast<const uint16_t*>(emb_bf16),
                     static_cast<const uint16_t*>(weight_bf16), static_cast<const uint16_t*>(bias_bf16), eps,
                     static_cast<half_t*>(out_f16));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // extern "C"
