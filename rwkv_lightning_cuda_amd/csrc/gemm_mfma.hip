// MFMA GEMM Y[M,N] = X[M,K] . W[N,K]^T for M >= 16: prefill chunks and batched decode.
//
// Reference: the cuBLAS / cuBLASLt calls behind rwkv7_v3a_linear_f16_orig_launch and
// rwkv7_v3a_linear_f16_orig_lt_cfg_launch (cuda/rwkv7_v3a_ops.cu:2235-2368) with the per-shape algorithm
// table of src/rwkv7_fast_v4.cu:753-958 -- fp16 inputs, fp32 accumulate, fp16 result.  The arithmetic lives
// in a closed library there; the contract restated here is the textbook GEMM with fp32 accumulation.
//
// gfx950 design.  v_mfma_f32_32x32x16_f16: lane l supplies 8 consecutive-k fp16 values of row l%32 of each
// operand (k half l/32), and X and W are both K-contiguous, so operands need no transpose: a lane reads
// them with plain 16-byte vector loads.  Per K tile of 64, lane (j = l%32, h = l/32) owns the 32 consecutive
// k values [32h, 32h+32) of weight row n0+j: 64 bytes of fp16, 32 bytes of int8 codes or 16 bytes of int4
// codes, expanded to fp16 in registers exactly (codes are small integers).  The X tile is staged in LDS
// (rows padded to keep 16-byte reads conflict-free) and shared by the four wavefronts of a block, each of
// which owns 32 output columns and all BM rows of the block tile.  W8 scales multiply the fp32 accumulator
// once in the epilogue; W4 accumulates sum (q - zp) x per 128-group in a second accumulator and folds it
// in with the group's scale, so no dequantised weight is rounded to fp16 -- the same arithmetic as the
// GEMV path.
#include "ops.h"

namespace rwkv {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kBK = 64;               // K tile
constexpr int kLdsStride = kBK + 8;   // fp16 elements per staged X row (pad 16 bytes)

struct GemmArgs {
  const half_t* x;
  const void* w;
  const half_t* scale;
  const uint8_t* zp;
  void* y;
  int M, N, K;
  int epilogue;
  int out_f32;
};

__device__ __forceinline__ half8_t make_half8(half2_t a, half2_t b, half2_t c, half2_t d) {
  half8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
  r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
  return r;
}

// 32 consecutive-k weights of one row as four MFMA B operands (8 fp16 each, exact).
template <int FMT>
__device__ __forceinline__ void load_b(const void* w, int64_t row, int K, int k, half8_t (&b)[4], int zp) {
  if constexpr (FMT == RWKV_FMT_F16) {
    const half_t* p = static_cast<const half_t*>(w) + row * K + k;
#pragma unroll
    for (int s = 0; s < 4; ++s) b[s] = *reinterpret_cast<const half8_t*>(p + 8 * s);
  } else if constexpr (FMT == RWKV_FMT_W8) {
    const int8_t* p = static_cast<const int8_t*>(w) + row * K + k;
    const uint4_t lo = *reinterpret_cast<const uint4_t*>(p);
    const uint4_t hi = *reinterpret_cast<const uint4_t*>(p + 16);
    const half2_t bias = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      // codes 8s..8s+7 = dwords 2s, 2s+1 of the 32-byte run
      const uint32_t d0 = ((s < 2) ? lo[(2 * s) & 3] : hi[(2 * s) & 3]) ^ 0x80808080u;
      const uint32_t d1 = ((s < 2) ? lo[(2 * s + 1) & 3] : hi[(2 * s + 1) & 3]) ^ 0x80808080u;
      b[s] = make_half8(as_half2(__builtin_amdgcn_perm(0x64646464u, d0, 0x04010400u)) - bias,
                        as_half2(__builtin_amdgcn_perm(0x64646464u, d0, 0x04030402u)) - bias,
                        as_half2(__builtin_amdgcn_perm(0x64646464u, d1, 0x04010400u)) - bias,
                        as_half2(__builtin_amdgcn_perm(0x64646464u, d1, 0x04030402u)) - bias);
    }
  } else {
    const uint8_t* p = static_cast<const uint8_t*>(w) + (row * K + k) / 2;
    const uint4_t q = *reinterpret_cast<const uint4_t*>(p);
    const float zf = 1024.0f + static_cast<float>(zp);
    const half2_t bias = {static_cast<half_t>(zf), static_cast<half_t>(zf)};  // exact: 1024..1039
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t d = q[s];  // 8 codes: element 2i in the low nibble of byte i
      const uint32_t even = d & 0x0f0f0f0fu;
      const uint32_t odd = (d >> 4) & 0x0f0f0f0fu;
      b[s] = make_half8(as_half2(__builtin_amdgcn_perm(odd, even, 0x0c040c00u) | 0x64006400u) - bias,
                        as_half2(__builtin_amdgcn_perm(odd, even, 0x0c050c01u) | 0x64006400u) - bias,
                        as_half2(__builtin_amdgcn_perm(odd, even, 0x0c060c02u) | 0x64006400u) - bias,
                        as_half2(__builtin_amdgcn_perm(odd, even, 0x0c070c03u) | 0x64006400u) - bias);
    }
  }
}

// grid = (ceil(N/128), ceil(M/BM)); block = 256 = 4 waves x 32 output columns; BM = 32*MB rows.
template <int FMT, int MB>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmArgs g) {
  constexpr int BM = 32 * MB;
  __shared__ __align__(16) half_t xs[BM * kLdsStride];

  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * 128 + wave * 32;
  const bool wave_active = n0 < g.N;
  const int n = min(n0 + j, g.N - 1);  // clamped: out-of-range columns compute garbage that is never stored
  const int K = g.K;

  float16_t acc[MB], part[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      acc[mb][v] = 0.0f;
      part[mb][v] = 0.0f;
    }

  for (int k0 = 0; k0 < K; k0 += kBK) {
    // weights for this tile first (independent of the staging barrier)
    half8_t b[4];
    int zp = 0;
    if constexpr (FMT == RWKV_FMT_W4) zp = g.zp[static_cast<int64_t>(n) * (K >> 7) + (k0 >> 7)];
    if (wave_active) load_b<FMT>(g.w, n, K, k0 + 32 * h, b, zp);

    __syncthreads();  // previous tile's readers are done
    // stage X[m0 .. m0+BM) x [k0, k0+64): 8 threads x 16 bytes per row
    for (int i = threadIdx.x; i < BM * 8; i += 256) {
      const int r = i >> 3;
      const int c = (i & 7) * 8;
      uint4_t val = {0u, 0u, 0u, 0u};
      if (m0 + r < g.M) val = *reinterpret_cast<const uint4_t*>(g.x + static_cast<int64_t>(m0 + r) * K + k0 + c);
      *reinterpret_cast<uint4_t*>(xs + r * kLdsStride + c) = val;
    }
    __syncthreads();

    if (wave_active) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const half8_t a = *reinterpret_cast<const half8_t*>(xs + (mb * 32 + j) * kLdsStride + 32 * h + 8 * s);
          if constexpr (FMT == RWKV_FMT_W4) {
            part[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[s], part[mb], 0, 0, 0);
          } else {
            acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b[s], acc[mb], 0, 0, 0);
          }
        }
      }
      if constexpr (FMT == RWKV_FMT_W4) {
        if (((k0 + kBK) & 127) == 0) {  // end of a 128-group: fold with the group's scale
          const float sc = h2f(g.scale[static_cast<int64_t>(n) * (K >> 7) + (k0 >> 7)]);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              acc[mb][v] = fmaf(part[mb][v], sc, acc[mb][v]);
              part[mb][v] = 0.0f;
            }
        }
      }
    }
  }
  if (!wave_active || n0 + j >= g.N) return;

  float sc = 1.0f;
  if constexpr (FMT == RWKV_FMT_W8) sc = h2f(g.scale[n]);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = m0 + mb * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
      if (row < g.M) {
        float val = round_h(acc[mb][v] * sc);
        if (g.epilogue == RWKV_EPI_RELU_SQUARE) {
          val = fmaxf(val, 0.0f);
          val = round_h(val * val);
        }
        const int64_t o = static_cast<int64_t>(row) * g.N + n;
        if (g.out_f32) {
          static_cast<float*>(g.y)[o] = val;
        } else {
          static_cast<half_t*>(g.y)[o] = f2h(val);
        }
      }
    }
  }
}

bool linear_mfma_supported(int fmt, int M, int N, int K) {
  if (M < 16 || N < 1 || K < kBK || K % kBK != 0) return false;
  if (fmt == RWKV_FMT_W4 && K % 128 != 0) return false;
  return fmt == RWKV_FMT_F16 || fmt == RWKV_FMT_W8 || fmt == RWKV_FMT_W4;
}

template <int FMT>
static int launch_fmt(hipStream_t st, const GemmArgs& g) {
  const int nblk = ceil_div(g.N, 128);
  // largest row tile that still leaves enough blocks to fill the 256 CUs
  int mb = 4;
  while (mb > 1 && (g.M <= 32 * (mb / 2) || nblk * ceil_div(g.M, 32 * mb) < 512)) mb /= 2;
  const dim3 grid(nblk, ceil_div(g.M, 32 * mb));
  switch (mb) {
    case 4: hipLaunchKernelGGL((gemm_mfma_kernel<FMT, 4>), grid, dim3(256), 0, st, g); break;
    case 2: hipLaunchKernelGGL((gemm_mfma_kernel<FMT, 2>), grid, dim3(256), 0, st, g); break;
    default: hipLaunchKernelGGL((gemm_mfma_kernel<FMT, 1>), grid, dim3(256), 0, st, g); break;
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int linear_mfma(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* w, const half_t* scale,
                const uint8_t* zp, int epilogue, int out_f32, void* y) {
  RWKV_REQUIRE(linear_mfma_supported(fmt, M, N, K), "linear_mfma: unsupported shape M=%d N=%d K=%d fmt=%d", M, N, K, fmt);
  RWKV_REQUIRE(x && w && y, "linear_mfma: NULL tensor");
  RWKV_REQUIRE(fmt == RWKV_FMT_F16 || scale, "linear_mfma: quantised weights need a scale tensor");
  RWKV_REQUIRE(fmt != RWKV_FMT_W4 || zp, "linear_mfma: W4 weights need a zero-point tensor");
  GemmArgs g;
  g.x = x; g.w = w; g.scale = scale; g.zp = zp; g.y = y; g.M = M; g.N = N; g.K = K;
  g.epilogue = epilogue; g.out_f32 = out_f32;
  switch (fmt) {
    case RWKV_FMT_W8: return launch_fmt<RWKV_FMT_W8>(st, g);
    case RWKV_FMT_W4: return launch_fmt<RWKV_FMT_W4>(st, g);
    default: return launch_fmt<RWKV_FMT_F16>(st, g);
  }
}

}  // namespace rwkv
