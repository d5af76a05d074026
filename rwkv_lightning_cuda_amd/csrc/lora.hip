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
// (w, a, g, v of a layer): grid = (C/128, row blocks, problems), block = 2 groups of 4 wavefronts x 32 output
// channels (the groups take alternate 16-wide steps of the rank and add up through LDS), the 32 x R slice of
// act(h) of a row tile staged in LDS.
#include <algorithm>
#include <cstdint>

#include "ops.h"

namespace rwkv {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kLoraMaxR = 512;
constexpr int kLoraRows = 32;   // rows per block: one MFMA tile
constexpr int kLoraCols = 128;  // output channels per block: 32 per wavefront
constexpr int kLoraKG = 2;       // wavefront groups that split the rank between them (even / odd 16-wide steps)
constexpr int kLoraThreads = 2 * kLoraCols * kLoraKG;
constexpr int kLoraStage = (kLoraRows * (kLoraMaxR / 8 + 1) + kLoraThreads - 1) / kLoraThreads;  // pieces per thread

// Per row tile: every lane requests its whole weight row (up to 16 pieces of 8; once per block - a block keeps
// its weights over all its row tiles), its pieces of the 32 x R hidden slice and its piece of the epilogue
// operands (v, v_first) in one go; the block turns the hidden slice into hi / lo fp16 in LDS (one barrier), each
// wavefront runs its MFMA steps, both groups lay their 32 x 128 sums out in LDS (over the hi / lo tiles, free by
// then) and all threads add the two in group order, apply the epilogue and write 16 bytes of a row each.
//
// Every load is issued without a per-lane branch around it: addresses past the rank or the last row are clamped to
// a valid one and the value is dropped afterwards.  (A load under a per-lane branch, or merged with a default
// value, makes the compiler wait for all loads in flight inside the branch: the trips to memory then run one
// after the other.)  Conditions that are the same for a whole wavefront cost nothing of the kind.
//
// LDS rows are R + 8 halves apart: for ranks that are multiples of 16 the ds_read_b128 of lane (j, h) at
// j * (2R + 16) + 16h bytes is conflict-free (other ranks lose some LDS bandwidth), and the zeroed 8-half pad is
// what the last MFMA step of a rank that is not a multiple of 16 reads (its weights are the clamped, finite ones).
constexpr int kLoraOutLd = kLoraCols + 4;  // fp32 row of the output tile in LDS

__global__ __launch_bounds__(kLoraThreads) void lora_out_kernel(LoraOutMultiArgs a) {
  __shared__ __attribute__((aligned(16))) half_t hi_s[kLoraRows * (kLoraMaxR + 8)];
  __shared__ __attribute__((aligned(16))) half_t lo_s[kLoraRows * (kLoraMaxR + 8)];
  static_assert(kLoraRows * kLoraOutLd * 4 <= kLoraRows * (kLoraMaxR + 8) * 2, "output tile exceeds the hidden tile");
  const LoraOutProblem& p = a.p[blockIdx.z];
  const int R = p.R;
  const int ld = R + 8;
  // wavefront-wide values, said so to the compiler: conditions on them become scalar branches
  const int wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3);
  const int kg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);  // its share of the rank: steps kg, kg + 2, ...
  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int c = blockIdx.x * kLoraCols + wave * 32 + j;
  const bool split = p.act != RWKV_ACT_NONE;
  const half_t* wrow = p.w2 + static_cast<int64_t>(c < a.C ? c : a.C - 1) * R;
  // packed weights: one 1 KiB piece per wavefront and rank step, consecutive lanes 16 bytes apart.  (Out of the
  // [C,R] matrix the 64 lanes of a request touch 64 different cache lines, and the address unit takes four times
  // as long over it.)
  const int steps = (R + 15) >> 4;
  const half_t* wpk = p.w2p ? p.w2p + (static_cast<int64_t>(blockIdx.x * (kLoraCols / 32) + wave) * steps * 64 + lane) * 8 : nullptr;

  // this lane's W2 values: k = 16*step + 8h .. +8 of output channel c
  constexpr int kSteps = kLoraMaxR / 16 / kLoraKG;
  half8_t w[kSteps];
#pragma unroll
  for (int i = 0; i < kSteps; ++i) {
    const int k0 = (i * kLoraKG + kg) * 16;  // the same for the whole wavefront
    if (k0 < R) {
      const int k = k0 + h * 8;
      w[i] = *reinterpret_cast<const half8_t*>(wpk ? wpk + static_cast<int64_t>(i * kLoraKG + kg) * 512 : wrow + (k < R ? k : R - 8));
    }
  }

  // the epilogue's view of the tile: thread t owns channels 8*(t%16) .. +8 of row t/16
  const int orow = threadIdx.x >> 4;
  const int ocol = blockIdx.x * kLoraCols + (threadIdx.x & 15) * 8;
  const bool ocol_ok = ocol < a.C;
  // without a bias any readable address does (C values of W2); the values are dropped in the epilogue
  uint4_t bias_raw = *reinterpret_cast<const uint4_t*>((p.bias ? p.bias : p.w2) + (ocol_ok ? ocol : 0));

  const int pieces = (R >> 3) + 1;  // R/8 pieces of 8 per row + the zeroed pad
  const int row_tiles = (a.M + kLoraRows - 1) / kLoraRows;
  auto row_tile = [&](int rt, bool more) {
    const int m0 = rt * kLoraRows;
    const int mn = min(kLoraRows, a.M - m0);
    uint4_t hv[kLoraStage];  // all of them loaded, whatever the rank: a value left undefined costs more than the load
#pragma unroll
    for (int i = 0; i < kLoraStage; ++i) {
      const int idx = threadIdx.x + i * kLoraThreads;
      const int m = idx / pieces;
      const int ks = (idx - m * pieces) * 8;
      hv[i] = *reinterpret_cast<const uint4_t*>(p.h + static_cast<int64_t>(m0 + (m < mn ? m : mn - 1)) * R +
                                                (ks < R ? ks : R - 8));
    }
    const int64_t o = static_cast<int64_t>(m0 + (orow < mn ? orow : mn - 1)) * a.C + (ocol_ok ? ocol : 0);
    // without the v-residual gate: the output row itself, readable and unused
    half8_t v8 = *reinterpret_cast<const half8_t*>((p.vres ? p.v : p.out) + o);
    half8_t vf8 = *reinterpret_cast<const half8_t*>((p.vres ? p.v_first : p.out) + o);
    __builtin_amdgcn_sched_barrier(0);
    // keeps the conversion of the bias below the loads above: moved up beside its own load, it would wait for the
    // weights before the hidden slice is even requested
    asm volatile("" : "+v"(bias_raw));
    const half8_t bias8 = __builtin_bit_cast(half8_t, bias_raw);

#pragma unroll
    for (int i = 0; i < kLoraStage; ++i) {
      if (i * kLoraThreads < kLoraRows * pieces) {
        const int idx = threadIdx.x + i * kLoraThreads;
        const int m = idx / pieces;
        const int ks = (idx - m * pieces) * 8;
        if (m < kLoraRows) {
          const bool live = m < mn && ks < R;  // rows past M and the pad hold exact zeros
          const half8_t raw = __builtin_bit_cast(half8_t, hv[i]);
          half8_t hi, lo;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            float f = h2f(raw[e]);
            if (p.act == RWKV_ACT_TANH) f = tanh_f(f);
            if (p.act == RWKV_ACT_SIGMOID) f = sigmoid_f(f);
            if (!live) f = 0.0f;
            hi[e] = f2h(f);
            lo[e] = f2h(f - h2f(hi[e]));
          }
          *reinterpret_cast<half8_t*>(&hi_s[m * ld + ks]) = hi;
          if (split) *reinterpret_cast<half8_t*>(&lo_s[m * ld + ks]) = lo;
        }
      }
    }
    __syncthreads();

    float16_t acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
    for (int i = 0; i < kSteps; ++i) {
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
    __syncthreads();  // the hidden tiles are free: group 0 lays its sums over hi_s, group 1 over lo_s
    // accumulator v of lane (j, h): row 8*(v/4) + 4h + v%4, column wave*32 + j
    float* tile = reinterpret_cast<float*>(kg == 0 ? hi_s : lo_s);
#pragma unroll
    for (int v = 0; v < 16; ++v) tile[(8 * (v / 4) + 4 * h + (v % 4)) * kLoraOutLd + wave * 32 + j] = acc[v];
    __syncthreads();

    const float* t0 = reinterpret_cast<const float*>(hi_s) + orow * kLoraOutLd + (threadIdx.x & 15) * 8;
    const float* t1 = reinterpret_cast<const float*>(lo_s) + orow * kLoraOutLd + (threadIdx.x & 15) * 8;
    float sum[8];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const float4_t s0 = *reinterpret_cast<const float4_t*>(t0 + 4 * q);
      const float4_t s1 = *reinterpret_cast<const float4_t*>(t1 + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) sum[4 * q + e] = s0[e] + s1[e];
    }
    half8_t res;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float b = p.bias ? h2f(bias8[e]) : 0.0f;
      if (p.vres) {
        const float vv = h2f(v8[e]);
        const float gate = sigmoid_f(b + sum[e]);
        res[e] = f2h(vv + (h2f(vf8[e]) - vv) * gate);
      } else {
        res[e] = f2h(sum[e] + b);
      }
    }
    if (orow < mn && ocol_ok) *reinterpret_cast<half8_t*>(p.out + o) = res;
    if (more) __syncthreads();  // the tiles are rewritten by the next row tile
  };
  // One tile per block (up to 256 rows) as straight-line code: inside a loop the compiler makes the requests of a
  // tile wait for the weights, for the sake of registers that the previous trip round the loop has long released.
  if (static_cast<int>(gridDim.y) >= row_tiles) {
    row_tile(blockIdx.y, false);
  } else {
    for (int rt = blockIdx.y; rt < row_tiles; rt += gridDim.y) row_tile(rt, true);
  }
}

// Row tiles per block: one up to 256 rows; beyond that the blocks of a problem walk the row tiles with a stride, so
// that the weights of a block are requested once for several tiles and the grid stays at a few blocks per CU.
__global__ __launch_bounds__(256) void lora_pack_w2_kernel(int C, int R, const half_t* __restrict__ w2, half_t* __restrict__ packed,
                                                           int64_t n_pieces) {
  const int64_t piece = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // (band, step, lane)
  if (piece >= n_pieces) return;
  const int steps = (R + 15) >> 4;
  const int lane = static_cast<int>(piece & 63);
  const int step = static_cast<int>((piece >> 6) % steps);
  const int band = static_cast<int>((piece >> 6) / steps);
  const int c = band * 32 + (lane & 31);
  const int k = step * 16 + (lane >> 5) * 8;
  half8_t v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = static_cast<half_t>(0.0f);
  if (c < C && k < R) v = *reinterpret_cast<const half8_t*>(w2 + static_cast<int64_t>(c) * R + k);  // R % 8 == 0
  *reinterpret_cast<half8_t*>(packed + piece * 8) = v;
}

// Whole column blocks of the rank-out kernel (kLoraCols channels = four 32-channel bands): the wavefronts of the
// last block read their bands without a clamp, so the bands past C exist and hold zeros.
size_t lora_pack_w2_halfs(int C, int R) {
  return static_cast<size_t>(ceil_div(C, kLoraCols)) * (kLoraCols / 32) * ((R + 15) >> 4) * 512;
}

int lora_pack_w2_launch(hipStream_t st, int C, int R, const half_t* w2, half_t* packed) {
  RWKV_REQUIRE(C > 0 && R > 0 && R % 8 == 0 && w2 && packed, "lora_pack_w2: bad arguments (C=%d, R=%d)", C, R);
  const int64_t n_pieces = static_cast<int64_t>(lora_pack_w2_halfs(C, R) / 8);
  hipLaunchKernelGGL(lora_pack_w2_kernel, dim3(static_cast<unsigned>((n_pieces + 255) / 256)), dim3(256), 0, st, C, R, w2, packed,
                     n_pieces);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
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
    RWKV_REQUIRE((reinterpret_cast<uintptr_t>(p.h) | reinterpret_cast<uintptr_t>(p.w2) | reinterpret_cast<uintptr_t>(p.out) |
                  reinterpret_cast<uintptr_t>(p.bias) | reinterpret_cast<uintptr_t>(p.v) |
                  reinterpret_cast<uintptr_t>(p.v_first) | reinterpret_cast<uintptr_t>(p.w2p)) % 16 == 0,
                 "lora_out: tensors must be 16-byte aligned");
  }
  const int row_tiles = ceil_div(a.M, kLoraRows);
  const int row_blocks = row_tiles <= 8 ? row_tiles : std::max(8, ceil_div(row_tiles, 8));
  hipLaunchKernelGGL(lora_out_kernel, dim3(ceil_div(a.C, kLoraCols), row_blocks, a.n), dim3(kLoraThreads), 0, st, a);
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
