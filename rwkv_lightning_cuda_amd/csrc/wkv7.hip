// WKV7 time-mix recurrence for gfx950, fp32 state.
//
// Reference semantics: cuda/rwkv7_wkv_fp32_v2.cu:100-126 (per token, thread i owns state row i):
//   sa = sum_j S[i][j]*a[j];  S[i][j] = S[i][j]*d[j] + sa*b[j] + k[j]*v[i];  y[i] = sum_j S[i][j]*r[j]
// with the decay map d = exp(-e^-1/2 * sigmoid(w)) of :13-14,26-28.
//
// Sequence kernel (any T): one wavefront per (batch, head); lane i keeps state row i in 64 VGPRs for
// the whole call.  The per-column operands r,d,k,a,b are the same for all 64 lanes, so they are read
// through the scalar cache into SGPRs (wave-uniform addresses) and feed the FMAs as scalar operands:
// no LDS traffic and no cross-lane work in the inner loop, and the summation order over j is the
// sequential one of the reference.  Operands must therefore be fp32 with the decay already applied;
// a small element-wise pre-pass produces them when the caller passes fp16 tensors or raw decay logits.
#include "ops.h"

namespace rwkv {

constexpr float kWScaleLog2e = -0.8750387749145276f;  // -e^-1/2 * log2(e), rwkv7_wkv_fp32_v2.cu:13
constexpr float kNLog2e = -1.4426950408889634f;       // rwkv7_wkv_fp32_v2.cu:14

__device__ __forceinline__ float decay_from_logit(float w) {
  return exp2f(kWScaleLog2e / (1.0f + exp2f(kNLog2e * w)));
}

// ---- pre-pass: any io type -> fp32 operands, decay applied -----------------------------------
// Source tensors are [B,T,C]; the pre-pass takes tokens [t0, t0+tn) of every batch row and writes
// compact fp32 [B,tn,C] operands.
template <typename IO>
__global__ __launch_bounds__(256) void wkv7_prepare_kernel(int64_t n, int64_t slab_row, int64_t src_row, int w_mode,
                                                           const IO* __restrict__ r, const IO* __restrict__ w,
                                                           const IO* __restrict__ k, const IO* __restrict__ a,
                                                           const IO* __restrict__ b, float* __restrict__ r32,
                                                           float* __restrict__ d32, float* __restrict__ k32,
                                                           float* __restrict__ a32, float* __restrict__ b32) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t bi = i / slab_row;            // slab_row = tn*C, src_row = T*C
  const int64_t src = bi * src_row + (i - bi * slab_row);
  const float wv = static_cast<float>(w[src]);
  r32[i] = static_cast<float>(r[src]);
  d32[i] = (w_mode == RWKV_W_RAW_LOGIT) ? decay_from_logit(wv) : wv;
  k32[i] = static_cast<float>(k[src]);
  a32[i] = static_cast<float>(a[src]);
  b32[i] = static_cast<float>(b[src]);
}

// ---- sequence kernel -------------------------------------------------------------------------
// grid = B*H, block = 64.  r,d,k,a,b: fp32, `op_bs` elements between batch rows, read with
// wave-uniform addresses; v,y: IO, `io_bs` elements between batch rows.  Runs T tokens.
template <typename IO>
__global__ __launch_bounds__(64) void wkv7_seq_kernel(int T, int C, int H, float* __restrict__ state,
                                                      const float* __restrict__ r, const float* __restrict__ d,
                                                      const float* __restrict__ k, const float* __restrict__ a,
                                                      const float* __restrict__ b, int64_t op_bs,
                                                      const IO* __restrict__ v, IO* __restrict__ y, int64_t io_bs) {
  const int bh = blockIdx.x;
  const int bi = bh / H;
  const int h = bh - bi * H;
  const int lane = threadIdx.x;
  float* srow = state + (static_cast<int64_t>(bh) * kHead + lane) * kHead;

  float S[kHead];
#pragma unroll
  for (int j = 0; j < kHead; j += 4) {
    const float4_t q = *reinterpret_cast<const float4_t*>(srow + j);
    S[j] = q.x; S[j + 1] = q.y; S[j + 2] = q.z; S[j + 3] = q.w;
  }

  int64_t base = static_cast<int64_t>(bi) * op_bs + h * kHead;  // wave-uniform
  int64_t iob = static_cast<int64_t>(bi) * io_bs + h * kHead + lane;
  float vi = static_cast<float>(v[iob]);
  for (int t = 0; t < T; ++t) {
    const float* __restrict__ ap = a + base;
    const float* __restrict__ bp = b + base;
    const float* __restrict__ dp = d + base;
    const float* __restrict__ kp = k + base;
    const float* __restrict__ rp = r + base;
    // prefetch the next token's v (per-lane) while this token computes
    float v_next = 0.0f;
    if (t + 1 < T) v_next = static_cast<float>(v[iob + C]);

    float sa = 0.0f;
#pragma unroll
    for (int j = 0; j < kHead; ++j) sa = fmaf(S[j], ap[j], sa);
    float yy = 0.0f;
#pragma unroll
    for (int j = 0; j < kHead; ++j) {
      float s = S[j];
      s = fmaf(s, dp[j], fmaf(sa, bp[j], kp[j] * vi));
      yy = fmaf(s, rp[j], yy);
      S[j] = s;
    }
    y[iob] = static_cast<IO>(yy);
    vi = v_next;
    base += C;
    iob += C;
  }

#pragma unroll
  for (int j = 0; j < kHead; j += 4) {
    float4_t q;
    q.x = S[j]; q.y = S[j + 1]; q.z = S[j + 2]; q.w = S[j + 3];
    *reinterpret_cast<float4_t*>(srow + j) = q;
  }
}

template <typename IO>
static int launch_wkv7(hipStream_t st, int B, int T, int C, int H, int w_mode, float* state, const IO* r,
                       const IO* w, const IO* k, const IO* v, const IO* a, const IO* b, IO* y) {
  const int64_t row = static_cast<int64_t>(T) * C;
  if (std::is_same<IO, float>::value && w_mode == RWKV_W_DECAY) {
    hipLaunchKernelGGL(wkv7_seq_kernel<IO>, dim3(B * H), dim3(64), 0, st, T, C, H, state,
                       reinterpret_cast<const float*>(r), reinterpret_cast<const float*>(w),
                       reinterpret_cast<const float*>(k), reinterpret_cast<const float*>(a),
                       reinterpret_cast<const float*>(b), row, v, y, row);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
  }
  // Pre-pass in slabs of tokens so the fp32 workspace stays bounded (5 operands x 256 MiB); the
  // state carries across slabs in HBM, which keeps the result bitwise independent of the slab size.
  const int64_t slab_budget = 64ll << 20;  // fp32 elements per operand
  const int t_slab = static_cast<int>(std::min<int64_t>(T, std::max<int64_t>(1, slab_budget / (static_cast<int64_t>(B) * C))));
  const int64_t slab_elems = static_cast<int64_t>(B) * t_slab * C;
  float* ws = nullptr;
  RWKV_HIP_TRY(hipMallocAsync(reinterpret_cast<void**>(&ws), sizeof(float) * 5 * slab_elems, st));
  float* r32 = ws;
  float* d32 = ws + slab_elems;
  float* k32 = ws + 2 * slab_elems;
  float* a32 = ws + 3 * slab_elems;
  float* b32 = ws + 4 * slab_elems;
  for (int t0 = 0; t0 < T; t0 += t_slab) {
    const int tn = std::min(t_slab, T - t0);
    const int64_t off = static_cast<int64_t>(t0) * C;
    const int64_t slab_row = static_cast<int64_t>(tn) * C;
    const int64_t n = slab_row * B;
    hipLaunchKernelGGL(wkv7_prepare_kernel<IO>, dim3(ceil_div(n, 256)), dim3(256), 0, st, n, slab_row, row, w_mode,
                       r + off, w + off, k + off, a + off, b + off, r32, d32, k32, a32, b32);
    hipLaunchKernelGGL(wkv7_seq_kernel<IO>, dim3(B * H), dim3(64), 0, st, tn, C, H, state, r32, d32, k32, a32, b32,
                       slab_row, v + off, y + off, row);
  }
  hipError_t err = hipGetLastError();
  hipError_t ferr = hipFreeAsync(ws, st);
  if (err != hipSuccess || ferr != hipSuccess) {
    set_error("wkv7 launch failed: %s", hipGetErrorString(err != hipSuccess ? err : ferr));
    return RWKV_E_RUNTIME;
  }
  return RWKV_OK;
}

int wkv7_seq_f16_launch(hipStream_t st, int B, int T, int C, int H, float* state, const float* r, const float* d,
                        const float* k, const float* a, const float* b, int64_t op_bs, const half_t* v, half_t* y,
                        int64_t io_bs) {
  hipLaunchKernelGGL(wkv7_seq_kernel<half_t>, dim3(B * H), dim3(64), 0, st, T, C, H, state, r, d, k, a, b, op_bs, v, y,
                     io_bs);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" int rwkv_hip_wkv7(rwkv_stream_t s, int B, int T, int C, int H, int w_mode, int io, void* state,
                             const void* r, const void* w, const void* k, const void* v, const void* a,
                             const void* b, void* y) {
  RWKV_REQUIRE(B > 0 && T > 0 && H > 0, "wkv7: B, T, H must be positive (got %d, %d, %d)", B, T, H);
  RWKV_REQUIRE(C == H * kHead, "wkv7: C (%d) must equal H*64 (%d)", C, H * kHead);
  RWKV_REQUIRE(w_mode == RWKV_W_RAW_LOGIT || w_mode == RWKV_W_DECAY, "wkv7: bad w_mode %d", w_mode);
  RWKV_REQUIRE(state && r && w && k && v && a && b && y, "wkv7: NULL tensor");
  if (io == RWKV_IO_F16) {
    return launch_wkv7<half_t>(as_stream(s), B, T, C, H, w_mode, static_cast<float*>(state),
                               static_cast<const half_t*>(r), static_cast<const half_t*>(w),
                               static_cast<const half_t*>(k), static_cast<const half_t*>(v),
                               static_cast<const half_t*>(a), static_cast<const half_t*>(b),
                               static_cast<half_t*>(y));
  }
  RWKV_REQUIRE(io == RWKV_IO_F32, "wkv7: bad io %d", io);
  return launch_wkv7<float>(as_stream(s), B, T, C, H, w_mode, static_cast<float*>(state),
                            static_cast<const float*>(r), static_cast<const float*>(w),
                            static_cast<const float*>(k), static_cast<const float*>(v),
                            static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(y));
}
