// LoRA pairs of the RWKV-7 time-mix block (decay w, in-context rate a, gate g, value residual v).
//
// Reference: rank-in cuda/rwkv7_v3a_ops.cu:813-940 (fp32 dot over C, fp16 hidden), rank-out
// :942-1130 (tanh / sigmoid applied to the fp16 hidden in fp32 and NOT re-rounded, fp32 dot over the
// rank, v-residual gate fused for the v group :1118-1123); unfused variants :209-367,685-811,1132-1270;
// dispatch src/rwkv7_fast_v4.cu:961-1014,1217-1260.
//
// rank-in is a plain small-N linear layer over fp16 weights [R,C] and reuses the GEMV / streaming GEMM kernels.
//
// rank-out is out[M,C] = act(h[M,R]) . W2[C,R]^T: a short reduction (R = 32..512) and many outputs, on
// v_mfma_f32_32x32x16_f16.  The activated hidden stays fp32 in the reference, so it enters the matrix core as
// two fp16 terms, hi = f16(a) and lo = f16(a - hi): hi + lo carries 22 bits of a, both products with the fp16
// weight are exact in fp32, and the result differs from an fp32 dot only by summation order.  Without an
// activation the hidden is fp16 already and the lo term is skipped.  One launch takes up to four problems
// (w, a, g, v of a layer): grid = (C/128, M/32, problems), block = 2 groups of 4 wavefronts x 32 output channels
// (the groups take alternate 16-wide steps of the rank and add up through LDS), the 32 x R slice of act(h)
// staged in LDS once per block.
#include "ops.h"

namespace rwkv {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kLoraMaxR = 512;
constexpr int kLoraRows = 32;   // rows per block: one MFMA tile
constexpr int kLoraCols = 128;  // output channels per block: 32 per wavefront
constexpr int kLoraKG = 2;       // wavefront groups that split the rank between them (even / odd 16-wide steps)
constexpr int kLoraThreads = 2 * kLoraCols * kLoraKG;
constexpr int kLoraStage = (kLoraRows * (kLoraMaxR / 8 + 1) + kLoraThreads - 1) / kLoraThreads;  // pieces per thread

// Every lane first requests its whole weight row (up to 32 pieces of 8), the block turns its 32 x R slice of the
// hidden into hi / lo fp16 in LDS while those loads are in flight (one barrier), then each wavefront runs its MFMA
// steps.  Rows are R + 8 halves apart:
// for ranks that are multiples of 16 the ds_read_b128 of lane (j, h) at j * (2R + 16) + 16h bytes is
// conflict-free (other ranks lose some LDS bandwidth), and the zeroed 8-half pad is what the last MFMA step of
// a rank that is not a multiple of 16 reads.
__global__ __launch_bounds__(kLoraThreads) void lora_out_kernel(LoraOutMultiArgs a) {
  __shared__ __attribute__((aligned(16))) half_t hi_s[kLoraRows * (kLoraMaxR + 8)];
  __shared__ __attribute__((aligned(16))) half_t lo_s[kLoraRows * (kLoraMaxR + 8)];
  const LoraOutProblem& p = a.p[blockIdx.z];
  const int R = p.R;
  const int ld = R + 8;
  const int m0 = blockIdx.y * kLoraRows;
  const int mn = min(kLoraRows, a.M - m0);
  const int wave = (threadIdx.x >> 6) & 3;
  const int kg = threadIdx.x >> 8;  // this wavefront's share of the rank: steps kg, kg + 2, ...
  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int c = blockIdx.x * kLoraCols + wave * 32 + j;
  const bool col_ok = c < a.C;
  const bool split = p.act != RWKV_ACT_NONE;
  const half_t* wrow = p.w2 + static_cast<int64_t>(col_ok ? c : 0) * R;

  // this lane's W2 values, all requested before the activation work: k = 16*kk + 8h .. +8 of output channel c
  half8_t w[kLoraMaxR / 16 / kLoraKG];
#pragma unroll
  for (int i = 0; i < kLoraMaxR / 16 / kLoraKG; ++i) {
    const int k = (i * kLoraKG + kg) * 16 + h * 8;
    if (k < R) {
      w[i] = *reinterpret_cast<const half8_t*>(wrow + k);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) w[i][e] = static_cast<half_t>(0.0f);
    }
  }

  // activation of the 32 x R hidden slice, split into hi + lo; R/8 pieces of 8 per row + the zeroed pad.  All of
  // a thread's pieces are requested before the first is used.
  const int pieces = (R >> 3) + 1;
  half8_t hv[kLoraStage];
#pragma unroll
  for (int i = 0; i < kLoraStage; ++i) {
    const int idx = threadIdx.x + i * kLoraThreads;
    const int m = idx / pieces;
    const int ks = (idx - m * pieces) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) hv[i][e] = static_cast<half_t>(0.0f);
    if (m < mn && ks < R) hv[i] = *reinterpret_cast<const half8_t*>(p.h + static_cast<int64_t>(m0 + m) * R + ks);
  }
#pragma unroll
  for (int i = 0; i < kLoraStage; ++i) {
    const int idx = threadIdx.x + i * kLoraThreads;
    const int m = idx / pieces;
    const int ks = (idx - m * pieces) * 8;
    if (m < kLoraRows) {
      half8_t hi, lo;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // rows past M and the pad hold zeros: every activation here maps them to values whose weights are zero
        // or whose rows are never stored, but the pad must be exactly zero
        float f = h2f(hv[i][e]);
        if (p.act == RWKV_ACT_TANH) f = tanh_f(f);
        if (p.act == RWKV_ACT_SIGMOID) f = sigmoid_f(f);
        if (ks >= R) f = 0.0f;
        hi[e] = f2h(f);
        lo[e] = f2h(f - h2f(hi[e]));
      }
      *reinterpret_cast<half8_t*>(&hi_s[m * ld + ks]) = hi;
      if (split) *reinterpret_cast<half8_t*>(&lo_s[m * ld + ks]) = lo;
    }
  }
  __syncthreads();

  float16_t acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
  for (int i = 0; i < kLoraMaxR / 16 / kLoraKG; ++i) {
    const int k = (i * kLoraKG + kg) * 16;
    if (k < R) {
      const half8_t ah = *reinterpret_cast<const half8_t*>(&hi_s[j * ld + k + h * 8]);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, w[i], acc, 0, 0, 0);
      if (split) {
        const half8_t al = *reinterpret_cast<const half8_t*>(&lo_s[j * ld + k + h * 8]);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, w[i], acc, 0, 0, 0);
      }
    }
  }
  // the second group's sums go through LDS (over the lo tile, which nobody reads any more) to the first
  __syncthreads();
  float* xch = reinterpret_cast<float*>(lo_s) + (wave * 64 + lane) * 16;
  if (kg == 1) {
#pragma unroll
    for (int v = 0; v < 16; v += 4) *reinterpret_cast<float4_t*>(xch + v) = float4_t{acc[v], acc[v + 1], acc[v + 2], acc[v + 3]};
  }
  __syncthreads();
  if (kg == 1) return;
#pragma unroll
  for (int v = 0; v < 16; v += 4) {
    const float4_t o = *reinterpret_cast<const float4_t*>(xch + v);
    acc[v] += o[0]; acc[v + 1] += o[1]; acc[v + 2] += o[2]; acc[v + 3] += o[3];
  }

  if (!col_ok) return;
  const float bias = p.bias ? h2f(p.bias[c]) : 0.0f;
  // accumulator v of lane (j, h): row 8*(v/4) + 4h + v%4, column j
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int m = 8 * (v / 4) + 4 * h + (v % 4);
    if (m < mn) {
      const int64_t o = static_cast<int64_t>(m0 + m) * a.C + c;
      float res;
      if (p.vres) {
        const float vv = h2f(p.v[o]);
        const float gate = sigmoid_f(bias + acc[v]);
        res = vv + (h2f(p.v_first[o]) - vv) * gate;
      } else {
        res = acc[v] + bias;
      }
      p.out[o] = f2h(res);
    }
  }
}

int lora_out_multi(hipStream_t st, const LoraOutMultiArgs& a) {
  RWKV_REQUIRE(a.n >= 1 && a.n <= 4, "lora_out: %d problems (1..4)", a.n);
  RWKV_REQUIRE(a.M > 0 && a.C > 0 && a.C % 32 == 0, "lora_out: C (%d) must be a positive multiple of 32", a.C);
  for (int i = 0; i < a.n; ++i) {
    const LoraOutProblem& p = a.p[i];
    RWKV_REQUIRE(p.R > 0 && p.R % 8 == 0 && p.R <= kLoraMaxR, "lora_out: rank %d must be a multiple of 8, at most %d",
                 p.R, kLoraMaxR);
    RWKV_REQUIRE(p.h && p.w2 && p.out, "lora_out: NULL tensor");
    RWKV_REQUIRE(!p.vres || (p.v && p.v_first && p.bias), "lora_out: v-residual gate needs v, v_first and v0");
  }
  hipLaunchKernelGGL(lora_out_kernel, dim3(ceil_div(a.C, kLoraCols), ceil_div(a.M, kLoraRows), a.n), dim3(kLoraThreads), 0, st,
                     a);
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
  LoraOutMultiArgs a = {};
  LoraOutProblem& p = a.p[0];
  p.h = static_cast<const half_t*>(h);
  p.w2 = static_cast<const half_t*>(w2);
  p.bias = static_cast<const half_t*>(bias);
  p.v = static_cast<const half_t*>(v);
  p.v_first = static_cast<const half_t*>(v_first);
  p.out = static_cast<half_t*>(out);
  p.R = R; p.act = act; p.vres = vres;
  a.n = 1; a.M = M; a.C = C;
  return lora_out_multi(as_stream(s), a);
}

}  // extern "C"
