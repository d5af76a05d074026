// Channel-mix down projection of a few tokens that reads, per token, only the rows of ffn.value whose activation
// is non-zero.
//
// Reference: rwkv7_cmix_sparse_down_relu_one_launch / _rows_launch and cmix_sparse_spmv_relu_one_kernel / _rows_kernel
// (cuda/rwkv7_fast_ops_fp16.cu:966-992,618-737; call site src/rwkv7_fast_v4.cu:1285-1292), per token:
//   vec[f] = f16(relu(preact[f])^2);  out[c] = sum over f with vec[f] != 0 of vec[f] * Wv[f][c]
// over ffn.value stored [F,C], so that a skipped f skips a contiguous row.  The reference accumulates in half2
// with atomicAdd (the result depends on block order); here the products are exact, the accumulation is fp32 and
// the order is fixed, so the result is the dense product of the same codes up to fp32 summation order.
//
// Weights: the [C,F] matrix transposed to [F,C]: fp16 values as they are, or int8 codes stored offset by 128
// (u = q + 128, one byte each) with the same per-output-channel fp16 scale.
//
// Kernel 1: grid = (F/256, column chunks, tokens), block = 8 wavefronts.  A wavefront owns 32 consecutive f and one 16-byte
// piece of the row per lane (1024 int8 or 512 fp16 columns per chunk): it ballots the non-zero activations, walks
// the set bits eight rows at a time (missing rows of the last batch repeat a row already read, with coefficient
// zero, so no load sits under a branch), and accumulates two rows per v_dot2_f32_f16: v_perm_b32 pairs the
// values of the two rows (int8: bytes under exponent 0x64, then one packed subtract gives the exact codes).  The eight wavefronts' sums meet in LDS in wavefront
// order and the block writes one fp32 partial row.  Kernel 2 sums the F/256 partial rows in a fixed order,
// applies the scale and rounds to fp16.
#include <mutex>

#include "ops.h"

namespace rwkv {

// Partial rows of the entry point that allocates nothing (rwkv_hip_cmix_sparse_down_relu_rows_static): a fixed
// array in the library's device image, one copy per GPU, held until the process ends.  In host code this name
// is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
constexpr size_t kStaticScratchBytes = static_cast<size_t>(16) << 20;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

constexpr int kSparseRowsPerWave = 32;
constexpr int kSparseWaves = 8;
constexpr int kSparseRowsPerBlock = kSparseRowsPerWave * kSparseWaves;  // 256
constexpr int kSparseBatch = 8;

// columns per lane = values in a 16-byte piece
constexpr int sparse_lane_cols(int fmt) { return fmt == RWKV_FMT_F16 ? 8 : 16; }

bool ffn_sparse_supported(int fmt, int C, int F) {
  if (fmt != RWKV_FMT_W8 && fmt != RWKV_FMT_F16 && fmt != RWKV_FMT_W4) return false;
  return C >= 16 && C % 16 == 0 && F >= kSparseRowsPerBlock && F % kSparseRowsPerBlock == 0;
}

// Bytes of the transposed copy.  int4: the [F,C/2] codes, then the scales [F/128,C] (fp16), then the zero points
// [F/128,C] (one byte each) - a wavefront's 32 rows lie in one 128-group, so it needs one scale and one zero point
// per column.
size_t ffn_sparse_packed_bytes(int fmt, int C, int F) {
  const size_t cf = static_cast<size_t>(C) * F;
  if (fmt == RWKV_FMT_F16) return cf * 2;
  if (fmt == RWKV_FMT_W8) return cf;
  return cf / 2 + static_cast<size_t>(F / 128) * C * 3;
}

size_t ffn_sparse_workspace_bytes(int rows, int C, int F) {
  return static_cast<size_t>(rows) * (F / kSparseRowsPerBlock) * C * sizeof(float);
}

// ---- [C,F] -> [F,C] (int8 codes get the offset) ----------------------------------------------------------------------
// grid = (F/64, C/64) tiles through LDS; C and F multiples of 64 are not required (edges are predicated).
template <typename E>
__global__ __launch_bounds__(256) void ffn_sparse_pack_kernel(int C, int F, const E* __restrict__ w, E* __restrict__ wt) {
  __shared__ E tile[64][65];
  const int f0 = blockIdx.x * 64;
  const int c0 = blockIdx.y * 64;
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int c = i >> 6;
    const int f = i & 63;
    E v = 0;
    if (c0 + c < C && f0 + f < F) v = w[static_cast<int64_t>(c0 + c) * F + f0 + f];
    if constexpr (sizeof(E) == 1) v ^= 0x80u;
    tile[c][f] = v;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    const int f = i >> 6;
    const int c = i & 63;
    if (c0 + c < C && f0 + f < F) wt[static_cast<int64_t>(f0 + f) * C + c0 + c] = tile[c][f];
  }
}

int ffn_sparse_pack_launch(hipStream_t st, int fmt, int C, int F, const void* w, void* wt) {
  RWKV_REQUIRE(fmt != RWKV_FMT_W4 && ffn_sparse_supported(fmt, C, F),
               "ffn_sparse_pack: unsupported format %d or shape C=%d F=%d (int4 codes: ffn_sparse_pack_w4)", fmt, C, F);
  RWKV_REQUIRE(w && wt && w != wt, "ffn_sparse_pack: bad pointers");
  const dim3 grid(ceil_div(F, 64), ceil_div(C, 64));
  if (fmt == RWKV_FMT_W8) {
    hipLaunchKernelGGL(ffn_sparse_pack_kernel<uint8_t>, grid, dim3(256), 0, st, C, F, static_cast<const uint8_t*>(w),
                       static_cast<uint8_t*>(wt));
  } else {
    hipLaunchKernelGGL(ffn_sparse_pack_kernel<uint16_t>, grid, dim3(256), 0, st, C, F, static_cast<const uint16_t*>(w),
                       static_cast<uint16_t*>(wt));
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// int4: q [C,F/2] (even f in the low nibble) -> t [F,C/2] (even c in the low nibble); 64 x 64 tiles of nibbles.
__global__ __launch_bounds__(256) void ffn_sparse_pack_w4_kernel(int C, int F, const uint8_t* __restrict__ q,
                                                                 uint8_t* __restrict__ t) {
  __shared__ uint8_t tile[64][65];
  const int f0 = blockIdx.x * 64;
  const int c0 = blockIdx.y * 64;
  for (int i = threadIdx.x; i < 64 * 32; i += 256) {
    const int c = i >> 5;
    const int fb = i & 31;
    uint8_t v = 0;
    if (c0 + c < C && f0 + 2 * fb < F) v = q[static_cast<int64_t>(c0 + c) * (F / 2) + f0 / 2 + fb];
    tile[c][2 * fb] = v & 15;
    tile[c][2 * fb + 1] = v >> 4;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 32; i += 256) {
    const int f = i >> 5;
    const int cb = i & 31;
    if (c0 + 2 * cb < C && f0 + f < F)
      t[static_cast<int64_t>(f0 + f) * (C / 2) + c0 / 2 + cb] = tile[2 * cb][f] | (tile[2 * cb + 1][f] << 4);
  }
}

// scale / zp [C,F/128] -> [F/128,C]
__global__ __launch_bounds__(256) void ffn_sparse_pack_w4_groups_kernel(int C, int G, const half_t* __restrict__ scale,
                                                                        const uint8_t* __restrict__ zp,
                                                                        half_t* __restrict__ scale_t,
                                                                        uint8_t* __restrict__ zp_t) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= static_cast<int64_t>(C) * G) return;
  const int g = static_cast<int>(i / C);
  const int c = static_cast<int>(i - static_cast<int64_t>(g) * C);
  scale_t[i] = scale[static_cast<int64_t>(c) * G + g];
  zp_t[i] = zp[static_cast<int64_t>(c) * G + g];
}

int ffn_sparse_pack_w4_launch(hipStream_t st, int C, int F, const void* q, const half_t* scale, const uint8_t* zp,
                              void* wt) {
  RWKV_REQUIRE(ffn_sparse_supported(RWKV_FMT_W4, C, F), "ffn_sparse_pack: unsupported shape C=%d F=%d", C, F);
  RWKV_REQUIRE(q && scale && zp && wt && q != wt, "ffn_sparse_pack: bad pointers");
  uint8_t* codes = static_cast<uint8_t*>(wt);
  const int G = F / 128;
  half_t* scale_t = reinterpret_cast<half_t*>(codes + static_cast<size_t>(C) * F / 2);
  uint8_t* zp_t = reinterpret_cast<uint8_t*>(scale_t + static_cast<size_t>(G) * C);
  hipLaunchKernelGGL(ffn_sparse_pack_w4_kernel, dim3(ceil_div(F, 64), ceil_div(C, 64)), dim3(256), 0, st, C, F,
                     static_cast<const uint8_t*>(q), codes);
  RWKV_LAUNCH_CHECK();
  hipLaunchKernelGGL(ffn_sparse_pack_w4_groups_kernel, dim3(static_cast<unsigned>((static_cast<int64_t>(C) * G + 255) / 256)),
                     dim3(256), 0, st, C, G, scale, zp, scale_t, zp_t);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// ---- kernel 1 ------------------------------------------------------------------------------------------------------------
// `activated` != 0: `in` already holds f16(relu(preact)^2) (the model's ffn.key launch applies it).
template <int FMT>
__global__ __launch_bounds__(64 * kSparseWaves) void ffn_sparse_kernel(int C, int F, int activated,
                                                                       const half_t* __restrict__ in,
                                                                       const uint4_t* __restrict__ wt,
                                                                       float* __restrict__ partial) {
  constexpr int LC = sparse_lane_cols(FMT);  // columns per lane
  constexpr int kCols = 64 * LC;             // columns per block
  __shared__ __align__(16) float red[kSparseWaves][kCols];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int f0 = blockIdx.x * kSparseRowsPerBlock + wave * kSparseRowsPerWave;
  const int c0 = blockIdx.y * kCols;
  const bool col_ok = c0 + LC * lane < C;
  // 16-byte pieces: row f has C/LC of them, this lane's piece of the row is (c0/LC + lane)
  const int row_pieces = C / LC;
  const uint4_t* wlane = wt + c0 / LC + (col_ok ? lane : 0);
  in += static_cast<int64_t>(blockIdx.z) * F;                       // this token's activations ...
  partial += static_cast<int64_t>(blockIdx.z) * gridDim.x * C;      // ... and partial rows

  float a = 0.0f;
  if (lane < kSparseRowsPerWave) {
    a = h2f(in[f0 + lane]);
    if (!activated) {
      a = fmaxf(round_h(a), 0.0f);
      a = round_h(a * a);
    }
  }
  const half_t ah = f2h(a);
  const uint32_t abits = __builtin_bit_cast(uint16_t, ah);
  uint64_t mask = __ballot((abits << 17) != 0u);  // +0 and -0 both count as zero

  float acc[LC];
#pragma unroll
  for (int i = 0; i < LC; ++i) acc[i] = 0.0f;
  const half2_t bias = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};

  while (mask != 0) {
    int row[kSparseBatch];
    uint32_t coef[kSparseBatch];
    const int first = __builtin_ctzll(mask);
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) {
      if (mask != 0) {
        row[p] = __builtin_ctzll(mask);
        mask &= mask - 1;
        coef[p] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits), row[p]));
      } else {
        row[p] = first;
        coef[p] = 0u;
      }
    }
    uint4_t q[kSparseBatch];
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) q[p] = __builtin_nontemporal_load(&wlane[static_cast<int64_t>(f0 + row[p]) * row_pieces]);
#pragma unroll
    for (int p = 0; p < kSparseBatch; p += 2) {
      const half2_t ap = as_half2(coef[p] | (coef[p + 1] << 16));
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t lo = q[p][d];
        const uint32_t hi = q[p + 1][d];
        if constexpr (FMT == RWKV_FMT_W8) {
          const half2_t w0 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c040c00u) | 0x64006400u) - bias;
          const half2_t w1 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c050c01u) | 0x64006400u) - bias;
          const half2_t w2 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c060c02u) | 0x64006400u) - bias;
          const half2_t w3 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c070c03u) | 0x64006400u) - bias;
          acc[4 * d + 0] = __builtin_amdgcn_fdot2(ap, w0, acc[4 * d + 0], false);
          acc[4 * d + 1] = __builtin_amdgcn_fdot2(ap, w1, acc[4 * d + 1], false);
          acc[4 * d + 2] = __builtin_amdgcn_fdot2(ap, w2, acc[4 * d + 2], false);
          acc[4 * d + 3] = __builtin_amdgcn_fdot2(ap, w3, acc[4 * d + 3], false);
        } else {
          // a dword holds two fp16 columns of a row: pair the low halves and the high halves of the two rows
          const half2_t w0 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x05040100u));
          const half2_t w1 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x07060302u));
          acc[2 * d + 0] = __builtin_amdgcn_fdot2(ap, w0, acc[2 * d + 0], false);
          acc[2 * d + 1] = __builtin_amdgcn_fdot2(ap, w1, acc[2 * d + 1], false);
        }
      }
    }
  }

#pragma unroll
  for (int i = 0; i < LC / 4; ++i)
    *reinterpret_cast<float4_t*>(&red[wave][LC * lane + 4 * i]) =
        float4_t{acc[4 * i], acc[4 * i + 1], acc[4 * i + 2], acc[4 * i + 3]};
  __syncthreads();
  if (threadIdx.x < kCols / 4) {
    const int c = 4 * threadIdx.x;
    float4_t sum = *reinterpret_cast<const float4_t*>(&red[0][c]);
#pragma unroll
    for (int w = 1; w < kSparseWaves; ++w) sum = sum + *reinterpret_cast<const float4_t*>(&red[w][c]);
    if (c0 + c < C) *reinterpret_cast<float4_t*>(partial + static_cast<int64_t>(blockIdx.x) * C + c0 + c) = sum;
  }
}

// int4 codes: the same walk with 8-byte pieces (16 columns per lane, 1024 per block).  The two rows of a
// v_dot2_f32_f16 are paired nibble by nibble: even and odd nibbles of each dword are masked into bytes, v_perm_b32
// puts row A's byte under exponent 0x64 in the low half and row B's in the high half, one packed subtract of
// 1024 gives the exact codes.  sum_f a_f (q_fc - zp_c) = sum_f a_f q_fc - zp_c sum_f a_f: the zero point and the
// scale of the wavefront's 128-group are applied once, after the walk.
__global__ __launch_bounds__(64 * kSparseWaves) void ffn_sparse_w4_kernel(int C, int F, int activated,
                                                                          const half_t* __restrict__ in,
                                                                          const uint8_t* __restrict__ blob,
                                                                          float* __restrict__ partial) {
  constexpr int LC = 16;
  constexpr int kCols = 64 * LC;
  __shared__ __align__(16) float red[kSparseWaves][kCols];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int f0 = blockIdx.x * kSparseRowsPerBlock + wave * kSparseRowsPerWave;
  const int c0 = blockIdx.y * kCols;
  const bool col_ok = c0 + LC * lane < C;
  const int cl = c0 + (col_ok ? LC * lane : 0);  // this lane's first column
  const int row_pieces = C / LC;                 // 8-byte pieces per row
  const uint2_t* wlane = reinterpret_cast<const uint2_t*>(blob) + cl / LC;
  const int G = F / 128;
  const half_t* scale_t = reinterpret_cast<const half_t*>(blob + static_cast<size_t>(C) * F / 2);
  const uint8_t* zp_t = reinterpret_cast<const uint8_t*>(scale_t + static_cast<size_t>(G) * C);
  const int64_t gat = static_cast<int64_t>(f0 / 128) * C + cl;
  const half8_t sc0 = *reinterpret_cast<const half8_t*>(scale_t + gat);
  const half8_t sc1 = *reinterpret_cast<const half8_t*>(scale_t + gat + 8);
  const uint4_t zq = *reinterpret_cast<const uint4_t*>(zp_t + gat);
  in += static_cast<int64_t>(blockIdx.z) * F;
  partial += static_cast<int64_t>(blockIdx.z) * gridDim.x * C;

  float a = 0.0f;
  if (lane < kSparseRowsPerWave) {
    a = h2f(in[f0 + lane]);
    if (!activated) {
      a = fmaxf(round_h(a), 0.0f);
      a = round_h(a * a);
    }
  }
  const half_t ah = f2h(a);
  const uint32_t abits = __builtin_bit_cast(uint16_t, ah);
  uint64_t mask = __ballot((abits << 17) != 0u);

  float acc[LC];
#pragma unroll
  for (int i = 0; i < LC; ++i) acc[i] = 0.0f;
  float asum = 0.0f;
  const half2_t bias = {static_cast<half_t>(1024.0f), static_cast<half_t>(1024.0f)};

  while (mask != 0) {
    int row[kSparseBatch];
    uint32_t coef[kSparseBatch];
    const int first = __builtin_ctzll(mask);
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) {
      if (mask != 0) {
        row[p] = __builtin_ctzll(mask);
        mask &= mask - 1;
        coef[p] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits), row[p]));
      } else {
        row[p] = first;
        coef[p] = 0u;
      }
    }
    uint2_t q[kSparseBatch];
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p)
      q[p] = __builtin_nontemporal_load(&wlane[static_cast<int64_t>(f0 + row[p]) * row_pieces]);
#pragma unroll
    for (int p = 0; p < kSparseBatch; p += 2) {
      const half2_t ap = as_half2(coef[p] | (coef[p + 1] << 16));
      asum += h2f(ap[0]) + h2f(ap[1]);
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const uint32_t lo = q[p][d];
        const uint32_t hi = q[p + 1][d];
        const uint32_t ea = lo & 0x0f0f0f0fu, oa = (lo >> 4) & 0x0f0f0f0fu;
        const uint32_t eb = hi & 0x0f0f0f0fu, ob = (hi >> 4) & 0x0f0f0f0fu;
        // nibble n of the dword is column 8 d + n: byte n / 2 of the even (n even) or odd word
        const half2_t w0 = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c040c00u) | 0x64006400u) - bias;
        const half2_t w1 = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c040c00u) | 0x64006400u) - bias;
        const half2_t w2 = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c050c01u) | 0x64006400u) - bias;
        const half2_t w3 = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c050c01u) | 0x64006400u) - bias;
        const half2_t w4 = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c060c02u) | 0x64006400u) - bias;
        const half2_t w5 = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c060c02u) | 0x64006400u) - bias;
        const half2_t w6 = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c070c03u) | 0x64006400u) - bias;
        const half2_t w7 = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c070c03u) | 0x64006400u) - bias;
        acc[8 * d + 0] = __builtin_amdgcn_fdot2(ap, w0, acc[8 * d + 0], false);
        acc[8 * d + 1] = __builtin_amdgcn_fdot2(ap, w1, acc[8 * d + 1], false);
        acc[8 * d + 2] = __builtin_amdgcn_fdot2(ap, w2, acc[8 * d + 2], false);
        acc[8 * d + 3] = __builtin_amdgcn_fdot2(ap, w3, acc[8 * d + 3], false);
        acc[8 * d + 4] = __builtin_amdgcn_fdot2(ap, w4, acc[8 * d + 4], false);
        acc[8 * d + 5] = __builtin_amdgcn_fdot2(ap, w5, acc[8 * d + 5], false);
        acc[8 * d + 6] = __builtin_amdgcn_fdot2(ap, w6, acc[8 * d + 6], false);
        acc[8 * d + 7] = __builtin_amdgcn_fdot2(ap, w7, acc[8 * d + 7], false);
      }
    }
  }

#pragma unroll
  for (int i = 0; i < LC; ++i) {
    const float zpf = static_cast<float>((zq[i >> 2] >> (8 * (i & 3))) & 0xffu);
    const float scf = h2f(i < 8 ? sc0[i] : sc1[i - 8]);
    acc[i] = (acc[i] - zpf * asum) * scf;
  }
#pragma unroll
  for (int i = 0; i < LC / 4; ++i)
    *reinterpret_cast<float4_t*>(&red[wave][LC * lane + 4 * i]) =
        float4_t{acc[4 * i], acc[4 * i + 1], acc[4 * i + 2], acc[4 * i + 3]};
  __syncthreads();
  if (threadIdx.x < kCols / 4) {
    const int c = 4 * threadIdx.x;
    float4_t sum = *reinterpret_cast<const float4_t*>(&red[0][c]);
#pragma unroll
    for (int w = 1; w < kSparseWaves; ++w) sum = sum + *reinterpret_cast<const float4_t*>(&red[w][c]);
    if (c0 + c < C) *reinterpret_cast<float4_t*>(partial + static_cast<int64_t>(blockIdx.x) * C + c0 + c) = sum;
  }
}

// ---- kernel 1 for several tokens at once ------------------------------------------------------------------------------
// TOK tokens share one walk: a wavefront ballots the rows that are non-zero for ANY of its tokens and reads each of
// them once; a token for which a row is zero takes it with coefficient zero (an exact zero product).  With a
// fraction z of zero activations per token the walk reads 1 - z^TOK of the matrix once, where one walk per token
// reads TOK * (1 - z) of it.  Per token the rows still add up in increasing order, but a token's rows pair up
// differently than in its own walk (a pair is one v_dot2), so the last bits of the fp32 sums can differ from the
// one-token kernel's; the result repeats bitwise from call to call.
template <int TOK>
__device__ __forceinline__ void sparse_union_heads(const half_t* __restrict__ in, int F, int f0, int lane, int activated,
                                                  uint32_t (&abits)[TOK], uint64_t& mask) {
  mask = 0;
#pragma unroll
  for (int t = 0; t < TOK; ++t) {
    float a = 0.0f;
    if (lane < kSparseRowsPerWave) {
      a = h2f(in[static_cast<int64_t>(t) * F + f0 + lane]);
      if (!activated) {
        a = fmaxf(round_h(a), 0.0f);
        a = round_h(a * a);
      }
    }
    const half_t ah = f2h(a);
    abits[t] = __builtin_bit_cast(uint16_t, ah);
    mask |= __ballot((abits[t] << 17) != 0u);  // +0 and -0 both count as zero
  }
}

// the wavefronts' sums of one token meet in LDS in wavefront order; the block writes the token's partial row
template <int LC>
__device__ __forceinline__ void sparse_block_row(const float (&acc)[LC], float (*red)[64 * LC], int wave, int lane, int C, int c0,
                                                 float* __restrict__ partial_row) {
  constexpr int kCols = 64 * LC;
#pragma unroll
  for (int i = 0; i < LC / 4; ++i)
    *reinterpret_cast<float4_t*>(&red[wave][LC * lane + 4 * i]) =
        float4_t{acc[4 * i], acc[4 * i + 1], acc[4 * i + 2], acc[4 * i + 3]};
  __syncthreads();
  if (threadIdx.x < kCols / 4) {
    const int c = 4 * threadIdx.x;
    float4_t sum = *reinterpret_cast<const float4_t*>(&red[0][c]);
#pragma unroll
    for (int w = 1; w < kSparseWaves; ++w) sum = sum + *reinterpret_cast<const float4_t*>(&red[w][c]);
    if (c0 + c < C) *reinterpret_cast<float4_t*>(partial_row + c0 + c) = sum;
  }
  __syncthreads();  // red is written again for the next token
}

template <int FMT, int TOK>
__global__ __launch_bounds__(64 * kSparseWaves) void ffn_sparse_union_kernel(int C, int F, int activated,
                                                                             const half_t* __restrict__ in,
                                                                             const uint4_t* __restrict__ wt,
                                                                             float* __restrict__ partial) {
  constexpr int LC = sparse_lane_cols(FMT);
  constexpr int kCols = 64 * LC;
  __shared__ __align__(16) float red[kSparseWaves][kCols];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int f0 = blockIdx.x * kSparseRowsPerBlock + wave * kSparseRowsPerWave;
  const int c0 = blockIdx.y * kCols;
  const bool col_ok = c0 + LC * lane < C;
  const int row_pieces = C / LC;
  const uint4_t* wlane = wt + c0 / LC + (col_ok ? lane : 0);

  uint32_t abits[TOK];
  uint64_t mask;
  sparse_union_heads<TOK>(in, F, f0, lane, activated, abits, mask);

  float acc[TOK][LC];
#pragma unroll
  for (int t = 0; t < TOK; ++t)
#pragma unroll
    for (int i = 0; i < LC; ++i) acc[t][i] = 0.0f;
  const half2_t bias = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};

  while (mask != 0) {
    int row[kSparseBatch];
    bool live[kSparseBatch];
    const int first = __builtin_ctzll(mask);
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) {
      live[p] = mask != 0;
      if (live[p]) {
        row[p] = __builtin_ctzll(mask);
        mask &= mask - 1;
      } else {
        row[p] = first;  // a row already read, taken with coefficient zero: no load sits under a branch
      }
    }
    uint4_t q[kSparseBatch];
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) q[p] = __builtin_nontemporal_load(&wlane[static_cast<int64_t>(f0 + row[p]) * row_pieces]);
#pragma unroll
    for (int p = 0; p < kSparseBatch; p += 2) {
      half2_t ap[TOK];
#pragma unroll
      for (int t = 0; t < TOK; ++t) {
        const uint32_t c0b = live[p] ? static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits[t]), row[p])) : 0u;
        const uint32_t c1b = live[p + 1] ? static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits[t]), row[p + 1])) : 0u;
        ap[t] = as_half2(c0b | (c1b << 16));
      }
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t lo = q[p][d];
        const uint32_t hi = q[p + 1][d];
        if constexpr (FMT == RWKV_FMT_W8) {
          const half2_t w0 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c040c00u) | 0x64006400u) - bias;
          const half2_t w1 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c050c01u) | 0x64006400u) - bias;
          const half2_t w2 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c060c02u) | 0x64006400u) - bias;
          const half2_t w3 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x0c070c03u) | 0x64006400u) - bias;
#pragma unroll
          for (int t = 0; t < TOK; ++t) {
            acc[t][4 * d + 0] = __builtin_amdgcn_fdot2(ap[t], w0, acc[t][4 * d + 0], false);
            acc[t][4 * d + 1] = __builtin_amdgcn_fdot2(ap[t], w1, acc[t][4 * d + 1], false);
            acc[t][4 * d + 2] = __builtin_amdgcn_fdot2(ap[t], w2, acc[t][4 * d + 2], false);
            acc[t][4 * d + 3] = __builtin_amdgcn_fdot2(ap[t], w3, acc[t][4 * d + 3], false);
          }
        } else {
          const half2_t w0 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x05040100u));
          const half2_t w1 = as_half2(__builtin_amdgcn_perm(hi, lo, 0x07060302u));
#pragma unroll
          for (int t = 0; t < TOK; ++t) {
            acc[t][2 * d + 0] = __builtin_amdgcn_fdot2(ap[t], w0, acc[t][2 * d + 0], false);
            acc[t][2 * d + 1] = __builtin_amdgcn_fdot2(ap[t], w1, acc[t][2 * d + 1], false);
          }
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TOK; ++t)
    sparse_block_row<LC>(acc[t], red, wave, lane, C, c0,
                         partial + (static_cast<int64_t>(t) * gridDim.x + blockIdx.x) * C);
}

// int4 codes, several tokens at once: the walk of ffn_sparse_w4_kernel over the union of the tokens' rows
template <int TOK>
__global__ __launch_bounds__(64 * kSparseWaves) void ffn_sparse_w4_union_kernel(int C, int F, int activated,
                                                                                const half_t* __restrict__ in,
                                                                                const uint8_t* __restrict__ blob,
                                                                                float* __restrict__ partial) {
  constexpr int LC = 16;
  constexpr int kCols = 64 * LC;
  __shared__ __align__(16) float red[kSparseWaves][kCols];
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int f0 = blockIdx.x * kSparseRowsPerBlock + wave * kSparseRowsPerWave;
  const int c0 = blockIdx.y * kCols;
  const bool col_ok = c0 + LC * lane < C;
  const int cl = c0 + (col_ok ? LC * lane : 0);
  const int row_pieces = C / LC;
  const uint2_t* wlane = reinterpret_cast<const uint2_t*>(blob) + cl / LC;
  const int G = F / 128;
  const half_t* scale_t = reinterpret_cast<const half_t*>(blob + static_cast<size_t>(C) * F / 2);
  const uint8_t* zp_t = reinterpret_cast<const uint8_t*>(scale_t + static_cast<size_t>(G) * C);
  const int64_t gat = static_cast<int64_t>(f0 / 128) * C + cl;
  const half8_t sc0 = *reinterpret_cast<const half8_t*>(scale_t + gat);
  const half8_t sc1 = *reinterpret_cast<const half8_t*>(scale_t + gat + 8);
  const uint4_t zq = *reinterpret_cast<const uint4_t*>(zp_t + gat);

  uint32_t abits[TOK];
  uint64_t mask;
  sparse_union_heads<TOK>(in, F, f0, lane, activated, abits, mask);

  float acc[TOK][LC];
  float asum[TOK];
#pragma unroll
  for (int t = 0; t < TOK; ++t) {
    asum[t] = 0.0f;
#pragma unroll
    for (int i = 0; i < LC; ++i) acc[t][i] = 0.0f;
  }
  const half2_t bias = {static_cast<half_t>(1024.0f), static_cast<half_t>(1024.0f)};

  while (mask != 0) {
    int row[kSparseBatch];
    bool live[kSparseBatch];
    const int first = __builtin_ctzll(mask);
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p) {
      live[p] = mask != 0;
      if (live[p]) {
        row[p] = __builtin_ctzll(mask);
        mask &= mask - 1;
      } else {
        row[p] = first;
      }
    }
    uint2_t q[kSparseBatch];
#pragma unroll
    for (int p = 0; p < kSparseBatch; ++p)
      q[p] = __builtin_nontemporal_load(&wlane[static_cast<int64_t>(f0 + row[p]) * row_pieces]);
#pragma unroll
    for (int p = 0; p < kSparseBatch; p += 2) {
      half2_t ap[TOK];
#pragma unroll
      for (int t = 0; t < TOK; ++t) {
        const uint32_t c0b = live[p] ? static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits[t]), row[p])) : 0u;
        const uint32_t c1b = live[p + 1] ? static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(abits[t]), row[p + 1])) : 0u;
        ap[t] = as_half2(c0b | (c1b << 16));
        asum[t] += h2f(ap[t][0]) + h2f(ap[t][1]);
      }
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const uint32_t lo = q[p][d];
        const uint32_t hi = q[p + 1][d];
        const uint32_t ea = lo & 0x0f0f0f0fu, oa = (lo >> 4) & 0x0f0f0f0fu;
        const uint32_t eb = hi & 0x0f0f0f0fu, ob = (hi >> 4) & 0x0f0f0f0fu;
        half2_t w[8];
        w[0] = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c040c00u) | 0x64006400u) - bias;
        w[1] = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c040c00u) | 0x64006400u) - bias;
        w[2] = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c050c01u) | 0x64006400u) - bias;
        w[3] = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c050c01u) | 0x64006400u) - bias;
        w[4] = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c060c02u) | 0x64006400u) - bias;
        w[5] = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c060c02u) | 0x64006400u) - bias;
        w[6] = as_half2(__builtin_amdgcn_perm(eb, ea, 0x0c070c03u) | 0x64006400u) - bias;
        w[7] = as_half2(__builtin_amdgcn_perm(ob, oa, 0x0c070c03u) | 0x64006400u) - bias;
#pragma unroll
        for (int t = 0; t < TOK; ++t)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[t][8 * d + i] = __builtin_amdgcn_fdot2(ap[t], w[i], acc[t][8 * d + i], false);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < TOK; ++t) {
#pragma unroll
    for (int i = 0; i < LC; ++i) {
      const float zpf = static_cast<float>((zq[i >> 2] >> (8 * (i & 3))) & 0xffu);
      const float scf = h2f(i < 8 ? sc0[i] : sc1[i - 8]);
      acc[t][i] = (acc[t][i] - zpf * asum[t]) * scf;
    }
    sparse_block_row<LC>(acc[t], red, wave, lane, C, c0,
                         partial + (static_cast<int64_t>(t) * gridDim.x + blockIdx.x) * C);
  }
}

// ---- kernel 2: out[c] = f16(scale[c] * sum of the partial rows); block 0 also does the optional row copy --------
// grid = (ceil(C/64), tokens), block = 256 = 16 groups of partial rows x 16 column quads.  Group g sums rows g, g+16, ... (its
// loads are independent, so they are all in flight together), the 16 group sums meet in LDS in group order.
__global__ __launch_bounds__(256) void ffn_sparse_finish_kernel(int C, int n_partial, const float* __restrict__ partial,
                                                                const half_t* __restrict__ scale,
                                                                half_t* __restrict__ out, RowCopy copy) {
  __shared__ __align__(16) float red[16][64];
  if (blockIdx.x == 0 && blockIdx.y == 0 && copy.n > 0) {
    for (int i = threadIdx.x * 8; i < copy.n; i += 256 * 8)
      *reinterpret_cast<uint4_t*>(copy.dst + i) = *reinterpret_cast<const uint4_t*>(copy.src + i);
  }
  const int g = threadIdx.x >> 4;
  const int cq = (threadIdx.x & 15) * 4;
  const int c = blockIdx.x * 64 + cq;
  partial += static_cast<int64_t>(blockIdx.y) * n_partial * C;  // this token's partial rows ...
  out += static_cast<int64_t>(blockIdx.y) * C;                  // ... and output row
  float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
  if (c < C) {
#pragma unroll 4
    for (int p = g; p < n_partial; p += 16) sum = sum + *reinterpret_cast<const float4_t*>(partial + static_cast<int64_t>(p) * C + c);
  }
  *reinterpret_cast<float4_t*>(&red[g][cq]) = sum;
  __syncthreads();
  if (threadIdx.x >= 16 || c >= C) return;
  float4_t total = *reinterpret_cast<const float4_t*>(&red[0][cq]);
#pragma unroll
  for (int i = 1; i < 16; ++i) total = total + *reinterpret_cast<const float4_t*>(&red[i][cq]);
  half4_t sv = {static_cast<half_t>(1.0f), static_cast<half_t>(1.0f), static_cast<half_t>(1.0f), static_cast<half_t>(1.0f)};
  if (scale) sv = *reinterpret_cast<const half4_t*>(scale + c);
  half4_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = f2h(total[i] * h2f(sv[i]));
  *reinterpret_cast<half4_t*>(out + c) = o;
}

template <int TOK>
static void launch_union(hipStream_t st, int fmt, dim3 grid, int C, int F, int activated, const half_t* in, const void* wt,
                         float* ws) {
  const dim3 block(64 * kSparseWaves);
  if (fmt == RWKV_FMT_W4) {
    hipLaunchKernelGGL((ffn_sparse_w4_union_kernel<TOK>), grid, block, 0, st, C, F, activated, in, static_cast<const uint8_t*>(wt), ws);
  } else if (fmt == RWKV_FMT_W8) {
    hipLaunchKernelGGL((ffn_sparse_union_kernel<RWKV_FMT_W8, TOK>), grid, block, 0, st, C, F, activated, in,
                       static_cast<const uint4_t*>(wt), ws);
  } else {
    hipLaunchKernelGGL((ffn_sparse_union_kernel<RWKV_FMT_F16, TOK>), grid, block, 0, st, C, F, activated, in,
                       static_cast<const uint4_t*>(wt), ws);
  }
}

int ffn_sparse_launch(hipStream_t st, int fmt, int rows, int C, int F, int activated, const half_t* in, const void* wt,
                      const half_t* scale, void* workspace, size_t workspace_bytes, half_t* out, const RowCopy* copy,
                      bool one_walk) {
  RWKV_REQUIRE(ffn_sparse_supported(fmt, C, F), "ffn_sparse: unsupported format %d or shape C=%d F=%d", fmt, C, F);
  RWKV_REQUIRE(rows >= 1 && rows <= kSparseMaxRows, "ffn_sparse: %d rows (1..%d)", rows, kSparseMaxRows);
  RWKV_REQUIRE(in && wt && out && (fmt != RWKV_FMT_W8 || scale), "ffn_sparse: NULL tensor");
  RWKV_REQUIRE(workspace && workspace_bytes >= ffn_sparse_workspace_bytes(rows, C, F),
               "ffn_sparse: workspace of %zu bytes needed, got %zu", ffn_sparse_workspace_bytes(rows, C, F), workspace_bytes);
  RowCopy cp;
  if (copy) {
    RWKV_REQUIRE(copy->n % 8 == 0, "ffn_sparse: row copy length %d must be a multiple of 8", copy->n);
    cp = *copy;
  }
  const int n_partial = F / kSparseRowsPerBlock;
  const dim3 grid(n_partial, ceil_div(C, 64 * sparse_lane_cols(fmt)), rows);
  if (one_walk && rows >= 2 && rows <= kSparseUnionMaxRows) {
    // the tokens share one walk over the rows that are non-zero for any of them
    const dim3 g2(grid.x, grid.y, 1);
    float* ws = static_cast<float*>(workspace);
    if (rows == 2) launch_union<2>(st, fmt, g2, C, F, activated, in, wt, ws);
    else if (rows == 3) launch_union<3>(st, fmt, g2, C, F, activated, in, wt, ws);
    else launch_union<4>(st, fmt, g2, C, F, activated, in, wt, ws);
  } else if (fmt == RWKV_FMT_W4) {
    hipLaunchKernelGGL(ffn_sparse_w4_kernel, grid, dim3(64 * kSparseWaves), 0, st, C, F, activated, in,
                       static_cast<const uint8_t*>(wt), static_cast<float*>(workspace));
  } else if (fmt == RWKV_FMT_W8) {
    hipLaunchKernelGGL(ffn_sparse_kernel<RWKV_FMT_W8>, grid, dim3(64 * kSparseWaves), 0, st, C, F, activated, in,
                       static_cast<const uint4_t*>(wt), static_cast<float*>(workspace));
  } else {
    hipLaunchKernelGGL(ffn_sparse_kernel<RWKV_FMT_F16>, grid, dim3(64 * kSparseWaves), 0, st, C, F, activated, in,
                       static_cast<const uint4_t*>(wt), static_cast<float*>(workspace));
  }
  RWKV_LAUNCH_CHECK();
  hipLaunchKernelGGL(ffn_sparse_finish_kernel, dim3(ceil_div(C, 64), rows), dim3(256), 0, st, C, n_partial,
                     static_cast<const float*>(workspace), fmt == RWKV_FMT_W8 ? scale : nullptr, out, cp);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_cmix_sparse_pack(rwkv_stream_t s, int fmt, int C, int F, const void* w, void* wt) {
  return ffn_sparse_pack_launch(as_stream(s), fmt, C, F, w, wt);
}

int rwkv_hip_cmix_sparse_pack_w4(rwkv_stream_t s, int C, int F, const void* q, const void* scale, const void* zp,
                                 void* wt) {
  return ffn_sparse_pack_w4_launch(as_stream(s), C, F, q, static_cast<const half_t*>(scale),
                                   static_cast<const uint8_t*>(zp), wt);
}

int rwkv_hip_cmix_sparse_packed_bytes(int fmt, int C, int F, size_t* bytes) {
  RWKV_REQUIRE(bytes, "cmix_sparse_packed_bytes: NULL argument");
  RWKV_REQUIRE(ffn_sparse_supported(fmt, C, F), "cmix_sparse_packed_bytes: unsupported format %d or shape C=%d F=%d", fmt, C,
               F);
  *bytes = ffn_sparse_packed_bytes(fmt, C, F);
  return RWKV_OK;
}

int rwkv_hip_cmix_sparse_workspace(int rows, int C, int F, size_t* bytes) {
  RWKV_REQUIRE(bytes, "cmix_sparse_workspace: NULL argument");
  RWKV_REQUIRE(ffn_sparse_supported(RWKV_FMT_W8, C, F), "cmix_sparse_workspace: unsupported shape C=%d F=%d", C, F);
  RWKV_REQUIRE(rows >= 1 && rows <= kSparseMaxRows, "cmix_sparse_workspace: %d rows (1..%d)", rows, kSparseMaxRows);
  *bytes = ffn_sparse_workspace_bytes(rows, C, F);
  return RWKV_OK;
}

int rwkv_hip_cmix_sparse_down_relu_rows(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                        const void* wt, const void* scale, void* workspace, size_t workspace_bytes,
                                        void* out) {
  return ffn_sparse_launch(as_stream(s), fmt, rows, C, F, 0, static_cast<const half_t*>(preact), wt,
                           static_cast<const half_t*>(scale), workspace, workspace_bytes, static_cast<half_t*>(out), nullptr, false);
}

int rwkv_hip_cmix_sparse_down_relu_rows_shared(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                               const void* wt, const void* scale, void* workspace,
                                               size_t workspace_bytes, void* out) {
  RWKV_REQUIRE(rows >= 2 && rows <= kSparseUnionMaxRows, "cmix_sparse_shared: %d rows (2..%d)", rows, kSparseUnionMaxRows);
  return ffn_sparse_launch(as_stream(s), fmt, rows, C, F, 0, static_cast<const half_t*>(preact), wt,
                           static_cast<const half_t*>(scale), workspace, workspace_bytes, static_cast<half_t*>(out), nullptr, true);
}

// Device address of this GPU's copy of `scratch`, looked up once per device (with that device current).
static int static_scratch_address(float** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static float* address[kMaxDevices] = {nullptr};
  int dev = 0;
  RWKV_HIP_TRY(hipGetDevice(&dev));
  RWKV_REQUIRE(dev >= 0 && dev < kMaxDevices, "cmix_sparse_static: device index %d out of range", dev);
  std::lock_guard<std::mutex> guard(lock);
  if (address[dev] == nullptr) {
    float* p = nullptr;
    RWKV_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
    RWKV_REQUIRE(p != nullptr, "cmix_sparse_static: no device address for the scratch array");
    address[dev] = p;
  }
  *out = address[dev];
  return RWKV_OK;
}

int rwkv_hip_cmix_sparse_down_relu_rows_static(rwkv_stream_t s, int fmt, int rows, int C, int F, const void* preact,
                                               const void* wt, const void* scale, void* out) {
  RWKV_REQUIRE(ffn_sparse_supported(fmt, C, F), "cmix_sparse_static: unsupported format %d or shape C=%d F=%d", fmt, C, F);
  RWKV_REQUIRE(rows >= 1 && rows <= kSparseMaxRows, "cmix_sparse_static: %d rows (1..%d)", rows, kSparseMaxRows);
  const size_t need = ffn_sparse_workspace_bytes(rows, C, F);
  RWKV_REQUIRE(need <= kStaticScratchBytes,
               "cmix_sparse_static: rows=%d C=%d F=%d needs %zu bytes of partial rows, the built-in scratch holds %zu", rows,
               C, F, need, kStaticScratchBytes);
  float* ws = nullptr;
  const int rc = static_scratch_address(&ws);
  if (rc != RWKV_OK) return rc;
  return ffn_sparse_launch(as_stream(s), fmt, rows, C, F, 0, static_cast<const half_t*>(preact), wt,
                           static_cast<const half_t*>(scale), ws, kStaticScratchBytes, static_cast<half_t*>(out), nullptr, false);
}

int rwkv_hip_cmix_sparse_down_relu_one(rwkv_stream_t s, int fmt, int C, int F, const void* preact, const void* wt,
                                       const void* scale, void* workspace, size_t workspace_bytes, void* out) {
  return rwkv_hip_cmix_sparse_down_relu_rows(s, fmt, 1, C, F, preact, wt, scale, workspace, workspace_bytes, out);
}

}  // extern "C"
