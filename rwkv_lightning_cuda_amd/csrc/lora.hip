// LoRA pairs of the RWKV-7 time-mix block (decay w, in-context rate a, gate g, value residual v).
//
// Reference: rank-in cuda/rwkv7_v3a_ops.cu:813-940 (fp32 dot over C, fp16 hidden), rank-out
// :942-1130 (tanh / sigmoid applied to the fp16 hidden in fp32 and NOT re-rounded, fp32 dot over the
// rank, v-residual gate fused for the v group :1118-1123); unfused variants :209-367,685-811,1132-1270;
// dispatch src/rwkv7_fast_v4.cu:961-1014,1217-1260.
//
// rank-in is a plain small-N linear layer over fp16 weights [R,C] and reuses the GEMV kernel.
// rank-out has a short reduction (R = 32..512) and many outputs: 8 lanes share one output channel,
// each lane keeps its slice of the W2 row in registers and walks the rows of the batch, so W2 is read
// once per block however many rows there are.
#include "ops.h"

namespace rwkv {

constexpr int kLoraMaxR = 512;
constexpr int kLoraRowsPerBlock = 16;


// grid = (C/32, ceil(M/16)); block = 256: 32 output channels x 8 lanes.
__global__ __launch_bounds__(256) void lora_out_kernel(LoraOutArgs a) {
  __shared__ float hs[kLoraRowsPerBlock][kLoraMaxR];
  const int R = a.R;
  const int m0 = blockIdx.y * kLoraRowsPerBlock;
  const int mn = min(kLoraRowsPerBlock, a.M - m0);
  for (int i = threadIdx.x; i < mn * R; i += 256) {
    const int m = i / R;
    const int r = i - m * R;
    float hv = h2f(a.h[static_cast<int64_t>(m0 + m) * R + r]);
    if (a.act == RWKV_ACT_TANH) hv = tanhf(hv);
    if (a.act == RWKV_ACT_SIGMOID) hv = sigmoid_f(hv);
    hs[m][r] = hv;
  }
  const int g = threadIdx.x & 7;
  const int c = blockIdx.x * 32 + (threadIdx.x >> 3);
  // this lane's slice of W2[c]: elements g*8 + 64*i + e
  half8_t wreg[kLoraMaxR / 64];
#pragma unroll
  for (int i = 0; i < kLoraMaxR / 64; ++i) {
    const int r0 = g * 8 + 64 * i;
    if (r0 < R) {
      wreg[i] = *reinterpret_cast<const half8_t*>(a.w2 + static_cast<int64_t>(c) * R + r0);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) wreg[i][e] = static_cast<half_t>(0.0f);
    }
  }
  __syncthreads();
  const float bias = a.bias ? h2f(a.bias[c]) : 0.0f;
  for (int m = 0; m < mn; ++m) {
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < kLoraMaxR / 64; ++i) {
      const int r0 = g * 8 + 64 * i;
      if (r0 < R) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc = fmaf(hs[m][r0 + e], h2f(wreg[i][e]), acc);
      }
    }
    acc = group_sum<8>(acc);
    if (g == 0) {
      const int64_t o = static_cast<int64_t>(m0 + m) * a.C + c;
      float res;
      if (a.vres) {
        const float vv = h2f(a.v[o]);
        const float gate = sigmoid_f(bias + acc);
        res = vv + (h2f(a.v_first[o]) - vv) * gate;
      } else {
        res = acc + bias;
      }
      a.out[o] = f2h(res);
    }
  }
}

int lora_out_launch(hipStream_t st, const LoraOutArgs& a) {
  RWKV_REQUIRE(a.M > 0 && a.C > 0 && a.C % 32 == 0, "lora_out: C (%d) must be a positive multiple of 32", a.C);
  RWKV_REQUIRE(a.R > 0 && a.R % 8 == 0 && a.R <= kLoraMaxR, "lora_out: rank %d must be a multiple of 8, at most %d",
               a.R, kLoraMaxR);
  RWKV_REQUIRE(a.h && a.w2 && a.out, "lora_out: NULL tensor");
  RWKV_REQUIRE(!a.vres || (a.v && a.v_first && a.bias), "lora_out: v-residual gate needs v, v_first and v0");
  hipLaunchKernelGGL(lora_out_kernel, dim3(a.C / 32, ceil_div(a.M, kLoraRowsPerBlock)), dim3(256), 0, st, a);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_lora_in(rwkv_stream_t s, int M, int C, int R, const void* x, const void* w1, void* h) {
  RWKV_REQUIRE(x && w1 && h, "lora_in: NULL tensor");
  return linear_any_m(as_stream(s), RWKV_FMT_F16, M, R, C, static_cast<const half_t*>(x), w1, nullptr, nullptr,
                      RWKV_EPI_NONE, 0, h);
}

int rwkv_hip_lora_out(rwkv_stream_t s, int M, int C, int R, int act, const void* h, const void* w2, const void* bias,
                      int vres, const void* v, const void* v_first, void* out) {
  RWKV_REQUIRE(act == RWKV_ACT_NONE || act == RWKV_ACT_TANH || act == RWKV_ACT_SIGMOID, "lora_out: bad act %d", act);
  LoraOutArgs a = {};
  a.h = static_cast<const half_t*>(h);
  a.w2 = static_cast<const half_t*>(w2);
  a.bias = static_cast<const half_t*>(bias);
  a.v = static_cast<const half_t*>(v);
  a.v_first = static_cast<const half_t*>(v_first);
  a.out = static_cast<half_t*>(out);
  a.M = M; a.C = C; a.R = R; a.act = act; a.vres = vres;
  return lora_out_launch(as_stream(s), a);
}

}  // extern "C"
