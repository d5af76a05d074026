// Linear layers y[M,N] = x[M,K] . W[N,K]^T for small M: weight-streaming GEMV kernels for fp16,
// W8A16 and W4A16 weights.
//
// Reference: cuda/rwkv7_v3a_ops.cu:464-560 (linear_orig_row1_exact_f16_kernel: one block per two
// output rows, half2 loads, fp32 accumulate) and the rows 2-4 family :369-462,562-683; dispatch in
// src/rwkv7_fast_v4.cu:709-959.
//
// gfx950 design: the work is HBM-bound, so each lane streams 16-byte weight vectors (global_load_dwordx4)
// with many loads in flight, x is staged once per block in LDS (re-read by every row), integer codes
// are expanded to fp16 in registers (v_perm_b32 + one packed fp16 add, exact) and accumulated against
// x with v_dot2_f32_f16 in fp32.  The per-row (W8) or per-128-group (W4) scale is applied to the fp32
// partial sums, so no dequantised weight is ever rounded to fp16.  One wavefront owns R output rows
// over the whole K range: no atomics, no cross-wave reduction, deterministic summation order.
#include "ops.h"

namespace rwkv {


struct LinearArgs {
  LinearProblem p[kMaxProblems];
  int K;
  int KT;        // K tile staged in LDS (multiple of the per-wave K step)
  int epilogue;
  int out_f32;
};

// 4 signed int8 codes in a dword -> two half2 (exact).  c ^ 0x80 is the code + 128 as an unsigned
// byte; 0x6400 | byte is the fp16 number 1024 + byte; subtracting 1152 leaves the code.
__device__ __forceinline__ void cvt_i8x4(uint32_t d, half2_t& lo, half2_t& hi) {
  const uint32_t u = d ^ 0x80808080u;
  const uint32_t l = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
  const uint32_t h = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
  const half2_t bias = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};
  lo = as_half2(l) - bias;
  hi = as_half2(h) - bias;
}

__device__ __forceinline__ float dot2(half2_t a, half2_t b, float c) {
  return __builtin_amdgcn_fdot2(a, b, c, false);
}

// fp32 partial dot of one 16-byte weight vector against the matching x slice (held as half2 pairs).
template <int FMT>
struct WeightVec;

template <>
struct WeightVec<RWKV_FMT_W8> {
  static constexpr int kElems = 16;  // weights per 16-byte load
  __device__ static __forceinline__ float dot(const uint4_t& wv, const half2_t* x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t lo, hi;
      cvt_i8x4(wv[i], lo, hi);
      acc = dot2(lo, x[2 * i], acc);
      acc = dot2(hi, x[2 * i + 1], acc);
    }
    return acc;
  }
};

template <>
struct WeightVec<RWKV_FMT_F16> {
  static constexpr int kElems = 8;
  __device__ static __forceinline__ float dot(const uint4_t& wv, const half2_t* x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = dot2(as_half2(wv[i]), x[i], acc);
    return acc;
  }
};

template <>
struct WeightVec<RWKV_FMT_W4> {
  static constexpr int kElems = 32;
  // returns sum_k code_k * x_k (codes 0..15, exact in fp16); the zero point is folded by the caller
  __device__ static __forceinline__ float dot(const uint4_t& wv, const half2_t* x, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t d = wv[i];
      const uint32_t even = d & 0x0f0f0f0fu;          // elements 0,2,4,6 of this dword
      const uint32_t odd = (d >> 4) & 0x0f0f0f0fu;    // elements 1,3,5,7
      const half2_t bias = {static_cast<half_t>(1024.0f), static_cast<half_t>(1024.0f)};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // half2 (element 2j, element 2j+1) = bytes j of `even` and `odd`, each OR 0x6400
        const uint32_t sel = 0x0c040c00u + j * 0x00010001u;
        const uint32_t pk = __builtin_amdgcn_perm(odd, even, sel) | 0x64006400u;
        acc = dot2(as_half2(pk) - bias, x[4 * i + j], acc);
      }
    }
    return acc;
  }
};

// grid = (ceil(maxN / (4*R)), n_problems); block = 256 (4 waves); dynamic LDS = M*KT*2 bytes.
template <int FMT, int M, int R>
__global__ __launch_bounds__(256) void linear_gemv_kernel(LinearArgs args) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  half_t* xs = reinterpret_cast<half_t*>(lds_raw);

  constexpr int E = WeightVec<FMT>::kElems;      // weights per lane per load
  constexpr int kStep = 64 * E;                  // K covered by one wave-wide load
  constexpr int kBytesPerRowNum = (FMT == RWKV_FMT_F16) ? 4 : (FMT == RWKV_FMT_W8 ? 2 : 1);  // bytes*2 per weight

  const LinearProblem prob = args.p[blockIdx.y];
  const int K = args.K;
  const int KT = args.KT;
  const int N = prob.N;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int row0 = (blockIdx.x * 4 + wave) * R;
  const bool active = row0 < N;
  const int64_t row_bytes = static_cast<int64_t>(K) * kBytesPerRowNum / 2;
  const unsigned char* wbase = static_cast<const unsigned char*>(prob.w) + static_cast<int64_t>(row0) * row_bytes;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

  for (int kt = 0; kt < K; kt += KT) {
    const int kn = min(KT, K - kt);
    if (kt > 0) __syncthreads();
    for (int i = threadIdx.x * 8; i < M * kn; i += 256 * 8) {
      const int m = i / kn;
      const int kk = i - m * kn;
      *reinterpret_cast<uint4_t*>(xs + m * KT + kk) =
          *reinterpret_cast<const uint4_t*>(prob.x + static_cast<int64_t>(m) * K + kt + kk);
    }
    __syncthreads();
    if (active) {
      for (int k0 = lane * E; k0 < kn; k0 += kStep) {
        uint4_t wv[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
          wv[r] = *reinterpret_cast<const uint4_t*>(wbase + r * row_bytes +
                                                    static_cast<int64_t>(kt + k0) * kBytesPerRowNum / 2);
        }
        if constexpr (FMT == RWKV_FMT_W4) {
          // 32 codes per lane all lie in one 128-group: scale and zero point are per (row, group)
          const int g = (kt + k0) >> 7;
          const int G = K >> 7;
#pragma unroll
          for (int m = 0; m < M; ++m) {
            half2_t xv[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint4_t t = *reinterpret_cast<const uint4_t*>(xs + m * KT + k0 + q * 8);
#pragma unroll
              for (int e = 0; e < 4; ++e) xv[q * 4 + e] = as_half2(t[e]);
            }
            float xsum = 0.0f;
            const half2_t ones = {static_cast<half_t>(1.0f), static_cast<half_t>(1.0f)};
#pragma unroll
            for (int e = 0; e < 16; ++e) xsum = dot2(xv[e], ones, xsum);
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const int64_t gi = static_cast<int64_t>(row0 + r) * G + g;
              const float sc = h2f(prob.scale[gi]);
              const float z = static_cast<float>(prob.zp[gi]);
              const float part = WeightVec<FMT>::dot(wv[r], xv, 0.0f) - z * xsum;
              acc[r][m] = fmaf(part, sc, acc[r][m]);
            }
          }
        } else {
          constexpr int XV = E / 2;  // half2 per lane per m
#pragma unroll
          for (int m = 0; m < M; ++m) {
            half2_t xv[XV];
#pragma unroll
            for (int q = 0; q < XV / 4; ++q) {
              const uint4_t t = *reinterpret_cast<const uint4_t*>(xs + m * KT + k0 + q * 8);
#pragma unroll
              for (int e = 0; e < 4; ++e) xv[q * 4 + e] = as_half2(t[e]);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][m] = WeightVec<FMT>::dot(wv[r], xv, acc[r][m]);
          }
        }
      }
    }
  }
  if (!active) return;

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);

  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = row0 + r;
      float sc = 1.0f;
      if constexpr (FMT == RWKV_FMT_W8) sc = h2f(prob.scale[n]);
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float v = round_h(acc[r][m] * sc);
        if (args.epilogue == RWKV_EPI_RELU_SQUARE) {
          v = fmaxf(v, 0.0f);
          v = round_h(v * v);
        }
        const int64_t o = static_cast<int64_t>(m) * N + n;
        if (args.out_f32) {
          static_cast<float*>(prob.y)[o] = v;
        } else {
          static_cast<half_t*>(prob.y)[o] = f2h(v);
        }
      }
    }
  }
}

template <int FMT, int M, int R>
static int launch_one(hipStream_t st, const LinearArgs& args, int n_problems, int max_n) {
  const size_t lds = static_cast<size_t>(M) * args.KT * sizeof(half_t);
  const dim3 grid(ceil_div(max_n, 4 * R), n_problems);
  hipLaunchKernelGGL((linear_gemv_kernel<FMT, M, R>), grid, dim3(256), lds, st, args);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

template <int FMT>
static int launch_fmt(hipStream_t st, const LinearArgs& args, int n_problems, int max_n, int M) {
  switch (M) {
    case 1: return launch_one<FMT, 1, 2>(st, args, n_problems, max_n);
    case 2: return launch_one<FMT, 2, 2>(st, args, n_problems, max_n);
    case 3: return launch_one<FMT, 3, 2>(st, args, n_problems, max_n);
    case 4: return launch_one<FMT, 4, 2>(st, args, n_problems, max_n);
    case 5: return launch_one<FMT, 5, 4>(st, args, n_problems, max_n);
    case 6: return launch_one<FMT, 6, 4>(st, args, n_problems, max_n);
    case 7: return launch_one<FMT, 7, 4>(st, args, n_problems, max_n);
    case 8: return launch_one<FMT, 8, 4>(st, args, n_problems, max_n);
    default: break;
  }
  set_error("linear: bad row tile %d", M);
  return RWKV_E_INVALID;
}

// Batched small-M linear: n_problems problems sharing fmt, M (<= 8), K, epilogue and output type.
int linear_small_m(hipStream_t st, int fmt, int M, int K, int n_problems, const LinearProblem* problems, int epilogue,
                   int out_f32) {
  RWKV_REQUIRE(M >= 1 && M <= 8, "linear_small_m: M %d out of range", M);
  RWKV_REQUIRE(n_problems >= 1 && n_problems <= kMaxProblems, "linear_small_m: %d problems", n_problems);
  const int elems = fmt == RWKV_FMT_F16 ? 8 : (fmt == RWKV_FMT_W8 ? 16 : 32);
  RWKV_REQUIRE(K > 0 && K % elems == 0, "linear: K (%d) must be a multiple of %d for this weight format", K, elems);
  if (fmt == RWKV_FMT_W4) RWKV_REQUIRE(K % 128 == 0, "linear: W4 needs K %% 128 == 0 (K = %d)", K);
  LinearArgs args;
  int max_n = 0;
  for (int i = 0; i < n_problems; ++i) {
    RWKV_REQUIRE(problems[i].N > 0 && problems[i].N % 4 == 0, "linear: N (%d) must be a positive multiple of 4",
                 problems[i].N);
    RWKV_REQUIRE(problems[i].w && problems[i].x && problems[i].y, "linear: NULL tensor");
    RWKV_REQUIRE(fmt == RWKV_FMT_F16 || problems[i].scale, "linear: quantised weights need a scale tensor");
    RWKV_REQUIRE(fmt != RWKV_FMT_W4 || problems[i].zp, "linear: W4 weights need a zero-point tensor");
    args.p[i] = problems[i];
    max_n = std::max(max_n, problems[i].N);
  }
  for (int i = n_problems; i < kMaxProblems; ++i) args.p[i] = problems[0];
  args.K = K;
  args.epilogue = epilogue;
  args.out_f32 = out_f32;
  // LDS tile of x: at most 32 KiB per block, a whole number of wave steps
  const int step = 64 * elems;
  int kt = (32768 / (2 * M)) / step * step;
  if (kt < step) kt = step;
  const int k_round = (K + step - 1) / step * step;
  args.KT = std::min(kt, k_round);
  switch (fmt) {
    case RWKV_FMT_F16: return launch_fmt<RWKV_FMT_F16>(st, args, n_problems, max_n, M);
    case RWKV_FMT_W8: return launch_fmt<RWKV_FMT_W8>(st, args, n_problems, max_n, M);
    case RWKV_FMT_W4: return launch_fmt<RWKV_FMT_W4>(st, args, n_problems, max_n, M);
    default: break;
  }
  set_error("linear: unknown weight format %d", fmt);
  return RWKV_E_INVALID;
}

// Any M: MFMA tiles when the shape allows it and M >= 16, else row tiles of <= 8 through the GEMV kernel.
int linear_any_m(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* w, const half_t* scale,
                 const uint8_t* zp, int epilogue, int out_f32, void* y) {
  RWKV_REQUIRE(M > 0, "linear: M must be positive");
  if (M >= 16 && linear_mfma_supported(fmt, M, N, K)) {
    return linear_mfma(st, fmt, M, N, K, x, w, scale, zp, epilogue, out_f32, y);
  }
  for (int m0 = 0; m0 < M; m0 += 8) {
    const int mt = std::min(8, M - m0);
    LinearProblem p;
    p.w = w;
    p.scale = scale;
    p.zp = zp;
    p.x = x + static_cast<int64_t>(m0) * K;
    p.y = out_f32 ? static_cast<void*>(static_cast<float*>(y) + static_cast<int64_t>(m0) * N)
                  : static_cast<void*>(static_cast<half_t*>(y) + static_cast<int64_t>(m0) * N);
    p.N = N;
    const int rc = linear_small_m(st, fmt, mt, K, 1, &p, epilogue, out_f32);
    if (rc != RWKV_OK) return rc;
  }
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" int rwkv_hip_linear(rwkv_stream_t s, int fmt, int M, int N, int K, const void* x, const void* w,
                               const void* scale, const void* zp, int epilogue, int out_f32, void* y) {
  RWKV_REQUIRE(epilogue == RWKV_EPI_NONE || epilogue == RWKV_EPI_RELU_SQUARE, "linear: bad epilogue %d", epilogue);
  return linear_any_m(as_stream(s), fmt, M, N, K, static_cast<const half_t*>(x), w,
                      static_cast<const half_t*>(scale), static_cast<const uint8_t*>(zp), epilogue, out_f32, y);
}
