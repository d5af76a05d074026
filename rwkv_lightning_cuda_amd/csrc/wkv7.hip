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
// grid = B*H, block = 64 (one wavefront per head): lane i owns row i of the 64x64 state in 64 VGPRs for the
// whole call.  r,d,k,a,b are fp32 with `op_bs` elements between batch rows; v,y are IO with `io_bs` elements
// between batch rows.  The five operand vectors of a token are the same for every lane, so they go through
// LDS: the wavefront stages them kSeqChunk tokens at a time with coalesced 16-byte loads (4 tokens x 256 bytes
// per load instruction), double-buffered, and each step reads them back as broadcast 16-byte LDS reads that
// the scheduler overlaps with the 256 FMAs of the step.  The loads of chunk c+1 are in flight while chunk c
// computes.  Each lane keeps its own v values of the chunk in registers.  The arithmetic of a step does not
// depend on the chunking, so splitting T over several calls is bitwise neutral.
constexpr int kSeqChunk = 8;

template <typename IO>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(1, 1))) void wkv7_seq_kernel(
    int T, int C, int H, float* __restrict__ state,
                                                      const float* __restrict__ r, const float* __restrict__ d,
                                                      const float* __restrict__ k, const float* __restrict__ a,
                                                      const float* __restrict__ b, int64_t op_bs,
                                                      const IO* __restrict__ v, IO* __restrict__ y, int64_t io_bs) {
  __shared__ __align__(16) float ops[2][5][kSeqChunk][kHead];  // [buffer][a,b,d,k,r][token][column]

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

  const int64_t base = static_cast<int64_t>(bi) * op_bs + h * kHead;
  const float* src[5] = {a + base, b + base, d + base, k + base, r + base};
  const int64_t iob = static_cast<int64_t>(bi) * io_bs + h * kHead + lane;
  const int st_tok = lane >> 4;        // staging: this lane's token within a group of 4 ...
  const int st_col = (lane & 15) * 4;  // ... and its 4 columns

  float4_t stage[5][kSeqChunk / 4];
  float v_next[kSeqChunk], v_cur[kSeqChunk];

  auto request = [&](int t0) {
#pragma unroll
    for (int o = 0; o < 5; ++o)
#pragma unroll
      for (int i = 0; i < kSeqChunk / 4; ++i) {
        const int t = t0 + st_tok + 4 * i;
        stage[o][i] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        if (t < T) stage[o][i] = *reinterpret_cast<const float4_t*>(src[o] + static_cast<int64_t>(t) * C + st_col);
      }
#pragma unroll
    for (int tt = 0; tt < kSeqChunk; ++tt) {
      v_next[tt] = 0.0f;
      if (t0 + tt < T) v_next[tt] = static_cast<float>(v[iob + static_cast<int64_t>(t0 + tt) * C]);
    }
  };
  auto commit = [&](int buf) {
#pragma unroll
    for (int o = 0; o < 5; ++o)
#pragma unroll
      for (int i = 0; i < kSeqChunk / 4; ++i)
        *reinterpret_cast<float4_t*>(&ops[buf][o][st_tok + 4 * i][st_col]) = stage[o][i];
#pragma unroll
    for (int tt = 0; tt < kSeqChunk; ++tt) v_cur[tt] = v_next[tt];
  };

  request(0);
  commit(0);
  __syncthreads();
  for (int t0 = 0; t0 < T; t0 += kSeqChunk) {
    const int buf = (t0 / kSeqChunk) & 1;
    const bool more = t0 + kSeqChunk < T;
    if (more) request(t0 + kSeqChunk);
    const int n = min(kSeqChunk, T - t0);
    // Operand reads are software-pipelined by hand (the compiler otherwise issues each LDS read right before
    // its use and stalls on every one): the a vector of a step and its first column group are requested during
    // the previous step; inside a step the reads of column group g+1 are issued before group g computes.
    // __builtin_amdgcn_sched_barrier(0) keeps the scheduler from sinking the reads back down.
    float4_t A[kHead / 4];
    float4_t G[2][8];  // per group of 8 columns: b, d, k, r as two float4 each
    auto load_a = [&](int tt, int lo, int hi) {
#pragma unroll
      for (int j4 = lo; j4 < hi; ++j4) A[j4] = *reinterpret_cast<const float4_t*>(&ops[buf][0][tt][4 * j4]);
    };
    auto load_group = [&](int tt, int g, float4_t (&dst)[8]) {
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        dst[2 * o] = *reinterpret_cast<const float4_t*>(&ops[buf][1 + o][tt][8 * g]);
        dst[2 * o + 1] = *reinterpret_cast<const float4_t*>(&ops[buf][1 + o][tt][8 * g + 4]);
      }
    };
    load_a(0, 0, kHead / 4);
    load_group(0, 0, G[0]);
#pragma unroll
    for (int tt = 0; tt < kSeqChunk; ++tt) {
      if (tt < n) {
        const float vi = v_cur[tt];
        float sa = 0.0f;
#pragma unroll
        for (int j4 = 0; j4 < kHead / 4; ++j4) {
          sa = fmaf(S[4 * j4 + 0], A[j4].x, sa);
          sa = fmaf(S[4 * j4 + 1], A[j4].y, sa);
          sa = fmaf(S[4 * j4 + 2], A[j4].z, sa);
          sa = fmaf(S[4 * j4 + 3], A[j4].w, sa);
        }
        float yy = 0.0f;
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          // requests for later use: next column group (or the next step's first one), a slice of the next a vector
          if (g + 1 < 8) {
            load_group(tt, g + 1, G[(g + 1) & 1]);
          } else if (tt + 1 < kSeqChunk) {
            load_group(tt + 1, 0, G[0]);
          }
          if (tt + 1 < kSeqChunk) load_a(tt + 1, 2 * g, 2 * g + 2);
          __builtin_amdgcn_sched_barrier(0);
          const float4_t(&q)[8] = G[g & 1];
          const float bb[8] = {q[0].x, q[0].y, q[0].z, q[0].w, q[1].x, q[1].y, q[1].z, q[1].w};
          const float dd[8] = {q[2].x, q[2].y, q[2].z, q[2].w, q[3].x, q[3].y, q[3].z, q[3].w};
          const float kk[8] = {q[4].x, q[4].y, q[4].z, q[4].w, q[5].x, q[5].y, q[5].z, q[5].w};
          const float rr[8] = {q[6].x, q[6].y, q[6].z, q[6].w, q[7].x, q[7].y, q[7].z, q[7].w};
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float sv = S[8 * g + e];
            sv = fmaf(sv, dd[e], fmaf(sa, bb[e], kk[e] * vi));
            yy = fmaf(sv, rr[e], yy);
            S[8 * g + e] = sv;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        y[iob + static_cast<int64_t>(t0 + tt) * C] = static_cast<IO>(yy);
      }
    }
    if (more) commit(buf ^ 1);
    __syncthreads();
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
