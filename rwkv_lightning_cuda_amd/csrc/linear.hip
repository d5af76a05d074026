// Linear layers y[M,N] = x[M,K] . W[N,K]^T for small M: weight-streaming GEMV kernels for fp16,
// W8A16 and W4A16 weights.
//
// Reference: cuda/rwkv7_v3a_ops.cu:464-560 (linear_orig_row1_exact_f16_kernel: one block per two
// output rows, half2 loads, fp32 accumulate) and the rows 2-4 family :369-462,562-683; dispatch in
// src/rwkv7_fast_v4.cu:709-959; the fused LoRA rank-in launches :813-940.
//
// gfx950 design: the work is HBM-bound, so each lane streams 16-byte weight vectors (global_load_dwordx4)
// and a wavefront keeps R*U of them in flight per lane (R output rows x U steps along K), double-buffered
// in registers so the next batch is requested before the current one is consumed.  The first batch is
// requested before x is staged in LDS, so the two latencies overlap.  Integer codes are expanded to fp16
// in registers (v_perm_b32 + one packed fp16 subtract, exact) and accumulated against x with
// v_dot2_f32_f16 in fp32.  The per-row (W8) or per-128-group (W4) scale is applied to the fp32 partial
// sums, so no dequantised weight is ever rounded to fp16.  One wavefront owns R output rows over the whole
// K range: no atomics, no cross-wave reduction, deterministic summation order.  Up to eight problems
// that share x-length K (r/k/v and the four LoRA rank-ins of a layer, in different weight formats) go out
// as one launch over a flattened block range.
#include <cstdlib>

#include "ops.h"

namespace rwkv {

struct LinearArgs {
  LinearProblem p[kMaxProblems];
  int block_end[kMaxProblems];  // exclusive prefix of blocks per problem
  int n_problems;
  int K;
  int KT;  // K tile staged in LDS (>= K when the whole x fits)
  int epilogue;
  int out_f32;
  LnPrologue ln;
  RowCopy copy;
};

// One row of the LayerNorm + lerp prologue into xs (K fp16 values).  Same two-pass statistics, explicit FMAs and
// rounding points as ln_fused_kernel (fused_ops.hip), and the same order of summation, so the result is
// bit-identical to running that kernel first: that kernel gives each of its 256, 512 or 1024 threads (by row
// length) one 8-element slice and adds wavefront sums in wavefront order; here thread t of 256 stands in for
// its threads t, t + 256, ... with one partial sum each, and the block sum walks the same list of wavefront sums
// (slots of absent threads hold zero, which changes no bit).  The fp32 row sum s = x + res lives in LDS (sbuf, K
// floats; each thread re-reads only what it wrote) instead of registers, so that the prologue does not cost the
// weight-streaming loop its occupancy.  256 threads; red holds 16 floats.
__device__ __forceinline__ float ln_block_sum4(float (&x)[4], float* red) {
#pragma unroll
  for (int j = 0; j < 4; ++j) x[j] = wave_sum_dpp(x[j]);
  __syncthreads();  // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) red[j * 4 + (threadIdx.x >> 6)] = x[j];
  }
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) t += red[i];
  return t;
}

template <int NW>
__device__ __forceinline__ void ln_prologue_row(const LnPrologue& ln, const half_t* mu, int K, int m, half_t* xs,
                                                float* sbuf, float* red, bool store) {
  static_assert(NW == 4, "the prologue mirrors the LayerNorm kernel with 256 threads");
  const int kend = K;
  const int64_t row = static_cast<int64_t>(m) * K;
  const int64_t xsrc = ln.mode == 2 ? ln.tokens[m] * static_cast<int64_t>(K) : row;
  float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = (threadIdx.x + 256 * j) * 8;
    if (c < kend) {
      const half8_t xv = *reinterpret_cast<const half8_t*>(ln.x + xsrc + c);
      float v[8];
      if (ln.mode == 1) {
        const half8_t rv = *reinterpret_cast<const half8_t*>(ln.res + row + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = h2f(xv[e]) + h2f(rv[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = h2f(xv[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[j] += v[e];
      *reinterpret_cast<float4_t*>(sbuf + c) = float4_t{v[0], v[1], v[2], v[3]};
      *reinterpret_cast<float4_t*>(sbuf + c + 4) = float4_t{v[4], v[5], v[6], v[7]};
    }
  }
  const float mean = ln_block_sum4(sum, red) / static_cast<float>(K);
  float sv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = (threadIdx.x + 256 * j) * 8;
    if (c < kend) {
      const float4_t lo = *reinterpret_cast<const float4_t*>(sbuf + c);
      const float4_t hi = *reinterpret_cast<const float4_t*>(sbuf + c + 4);
      const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[e] - mean;
        sv[j] = fmaf(d, d, sv[j]);
      }
    }
  }
  const float sv_total = ln_block_sum4(sv, red);
  const float rstd = rsqrtf(sv_total / static_cast<float>(K) + ln.eps);
#pragma unroll 1
  for (int c = threadIdx.x * 8; c < kend; c += 256 * 8) {
    const half8_t wv = *reinterpret_cast<const half8_t*>(ln.w + c);
    const half8_t bv = *reinterpret_cast<const half8_t*>(ln.b + c);
    const half8_t pv = *reinterpret_cast<const half8_t*>(ln.shift + row + c);
    const half8_t mv = *reinterpret_cast<const half8_t*>(mu + c);
    const float4_t lo = *reinterpret_cast<const float4_t*>(sbuf + c);
    const float4_t hi = *reinterpret_cast<const float4_t*>(sbuf + c + 4);
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    half8_t yv, ov;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      yv[e] = f2h(fmaf((v[e] - mean) * rstd, h2f(wv[e]), h2f(bv[e])));
      const float yf = h2f(yv[e]);  // the lerp reads the fp16-rounded LN output
      ov[e] = f2h(fmaf(h2f(pv[e]) - yf, h2f(mv[e]), yf));
    }
    *reinterpret_cast<half8_t*>(xs + c) = ov;
    if (store) {
      *reinterpret_cast<half8_t*>(ln.ln_out + row + c) = yv;
      if (ln.x_out) {
        half8_t xo;
#pragma unroll
        for (int e = 0; e < 8; ++e) xo[e] = f2h(v[e]);
        *reinterpret_cast<half8_t*>(ln.x_out + row + c) = xo;
      }
    }
  }
}

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
  // sum_k (code_k - zp) * x_k over the lane's 32 codes (all in one 128-group), exact products.  A dword holds
  // elements 0..7 as nibbles n0..n7; (d >> 4j) & 0x000f000f picks (n_j, n_{j+4}), OR 0x6400 makes them the fp16
  // numbers 1024 + code, one packed subtract of 1024 + zp leaves code - zp.  xp[4i + j] must hold
  // (x_{8i+j}, x_{8i+j+4}).
  __device__ static __forceinline__ float dot(const uint4_t& wv, const half2_t* xp, half2_t zb, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t d = wv[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t pk = ((d >> (4 * j)) & 0x000f000fu) | 0x64006400u;
        acc = dot2(as_half2(pk) - zb, xp[4 * i + j], acc);
      }
    }
    return acc;
  }
  // (x0,x1)(x2,x3)(x4,x5)(x6,x7) per 8 elements -> (x0,x4)(x1,x5)(x2,x6)(x3,x7)
  __device__ static __forceinline__ void pair_x(const half2_t* xv, half2_t* xp) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = __builtin_bit_cast(uint32_t, xv[4 * i + j / 2]);
        const uint32_t hi = __builtin_bit_cast(uint32_t, xv[4 * i + 2 + j / 2]);
        xp[4 * i + j] = as_half2(__builtin_amdgcn_perm(hi, lo, (j & 1) ? 0x07060302u : 0x05040100u));
      }
    }
  }
};

// ---- int4 codes in the whole-rows-in-flight kernel ------------------------------------------------------------------
// A block whose weights are int4 codes keeps x in LDS in the order the nibble pairs want it - every 8 values
// (x0..x7) as (x0,x4)(x1,x5)(x2,x6)(x3,x7) - and, beside it, the fp32 sum of every 32 values (one lane's slice, inside
// one 128-group).  A nibble pair (n_j, n_{j+4}) of a dword is shifted into the top four mantissa bits of two fp16
// numbers with the exponent of 16: 0x4c00 | n << 6 is 16 + n, exactly.  Then
//   sum_k (q_k - zp) x_k = sum_k (16 + q_k) x_k - (16 + zp) sum_k x_k:
// the zero point and the offset leave in one multiply-add per slice instead of one packed subtract per pair, and
// x needs no pairing per wavefront (per 16-byte vector of 32 codes: 28 shift / mask instructions and 16 v_dot2
// where the pairing, the subtracts and the masks were 72).  Products (16 + q) x are exact in fp32; the offset is
// small against the terms (at most 31 |x| each), so nothing is lost to cancellation.
__device__ __forceinline__ uint4_t w4_pair_order(uint4_t v) {
  uint4_t o;
  o[0] = __builtin_amdgcn_perm(v[2], v[0], 0x05040100u);
  o[1] = __builtin_amdgcn_perm(v[2], v[0], 0x07060302u);
  o[2] = __builtin_amdgcn_perm(v[3], v[1], 0x05040100u);
  o[3] = __builtin_amdgcn_perm(v[3], v[1], 0x07060302u);
  return o;
}

// fp32 sum of the 32 values that four neighbouring lanes hold eight each (in every one of the four lanes)
__device__ __forceinline__ float w4_slice_sum(uint4_t v) {
  const half2_t a = as_half2(v[0]), b = as_half2(v[1]), c = as_half2(v[2]), d = as_half2(v[3]);
  float s = ((h2f(a[0]) + h2f(a[1])) + (h2f(b[0]) + h2f(b[1]))) + ((h2f(c[0]) + h2f(c[1])) + (h2f(d[0]) + h2f(d[1])));
  s = dpp_add<0xB1>(s);  // quad_perm [1,0,3,2]
  s = dpp_add<0x4E>(s);  // quad_perm [2,3,0,1]
  return s;
}

// (v & 0x03c003c0) | 0x4c004c00 as one v_bfi_b32 - the mask picks v's bits, the rest comes from the constant; the
// compiler emits the and and the or apart (v_and_or_b32 takes no two literals on this target)
__device__ __forceinline__ uint32_t w4_mask_or(uint32_t v) {
  uint32_t d;
  asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "s"(0x03c003c0u), "v"(v), "v"(0x4c004c00u));
  return d;
}

// sum_k (16 + code_k) x_k over a lane's 32 codes; xp[4i + j] holds (x_{8i+j}, x_{8i+j+4})
__device__ __forceinline__ float w4_dot_offset16(const uint4_t& wv, const half2_t* xp, float acc) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t d = wv[i];
    const uint32_t p0 = w4_mask_or(d << 6);
    const uint32_t p1 = w4_mask_or(d << 2);
    const uint32_t p2 = w4_mask_or(d >> 2);
    const uint32_t p3 = w4_mask_or(d >> 6);
    acc = dot2(as_half2(p0), xp[4 * i + 0], acc);
    acc = dot2(as_half2(p1), xp[4 * i + 1], acc);
    acc = dot2(as_half2(p2), xp[4 * i + 2], acc);
    acc = dot2(as_half2(p3), xp[4 * i + 3], acc);
  }
  return acc;
}

template <int FMT>
struct FmtTraits {
  static constexpr int kElems = WeightVec<FMT>::kElems;
  static constexpr int kStep = 64 * kElems;  // K covered by one wave-wide load
  // byte offset of element k within a row
  __device__ static __forceinline__ int64_t byte_off(int64_t k) {
    return FMT == RWKV_FMT_F16 ? k * 2 : (FMT == RWKV_FMT_W8 ? k : k / 2);
  }
};

// One wave: R rows of `prob`, K range [k_lo, k_lo + kn) whose x lives in LDS at xs[m*KT + k - k_lo].
template <int FMT, int M, int R, int U>
struct WaveGemv {
  using T = FmtTraits<FMT>;

  // One batch of weight vectors in flight; for int4 codes also the (row, 128-group) scale and zero point of each
  // vector (the lane's 32 codes all lie in one group), requested together with it.
  struct Batch {
    uint4_t w[U][R];
    half_t sc[U][R];
    uint8_t zp[U][R];
  };

  __device__ static __forceinline__ void load_batch(Batch& bt, const unsigned char* wbase, int64_t row_bytes, int k_lo, int kn,
                                                    int step0, int lane, const LinearProblem& prob, int row0, int K) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = (step0 + u) * T::kStep + lane * T::kElems;
      if (k0 < kn) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          // streamed once per step: non-temporal, so that the weights do not push the rows that are re-read (LoRA
          // matrices, state, activations) out of the caches (batch-1 step 2.39 -> 2.34 ms)
          bt.w[u][r] = __builtin_nontemporal_load(
              reinterpret_cast<const uint4_t*>(wbase + r * row_bytes + T::byte_off(k_lo + k0)));
          if constexpr (FMT == RWKV_FMT_W4) {
            const int64_t gi = static_cast<int64_t>(row0 + r) * (K >> 7) + ((k_lo + k0) >> 7);
            bt.sc[u][r] = prob.scale[gi];
            bt.zp[u][r] = prob.zp[gi];
          }
        }
      }
    }
  }

  __device__ static __forceinline__ void compute_batch(float (&acc)[R][M], const Batch& bt, const half_t* xs, int KT,
                                                       int kn, int step0, int lane) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = (step0 + u) * T::kStep + lane * T::kElems;
      if (k0 < kn) {
        constexpr int XV = T::kElems / 2;  // half2 per lane per m
#pragma unroll
        for (int m = 0; m < M; ++m) {
          half2_t xv[XV];
#pragma unroll
          for (int q = 0; q < XV / 4; ++q) {
            const uint4_t t = *reinterpret_cast<const uint4_t*>(xs + m * KT + k0 + q * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) xv[q * 4 + e] = as_half2(t[e]);
          }
          if constexpr (FMT == RWKV_FMT_W4) {
            half2_t xp[XV];
            WeightVec<FMT>::pair_x(xv, xp);
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const half_t zf = static_cast<half_t>(1024.0f + static_cast<float>(bt.zp[u][r]));
              const half2_t zb = {zf, zf};
              const float part = WeightVec<FMT>::dot(bt.w[u][r], xp, zb, 0.0f);
              acc[r][m] = fmaf(part, h2f(bt.sc[u][r]), acc[r][m]);
            }
          } else {
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][m] = WeightVec<FMT>::dot(bt.w[u][r], xv, acc[r][m]);
          }
        }
      }
    }
  }
};

template <int FMT, int M, int R, int U, bool LN, int NW>
__device__ __forceinline__ void gemv_block(const LinearArgs& args, const LinearProblem& prob, int block_in_problem,
                                           half_t* xs, float* sbuf, float* red) {
  using T = FmtTraits<FMT>;
  using W = WaveGemv<FMT, M, R, U>;
  const int K = args.K;
  const int KT = args.KT;
  const int N = prob.N;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int row0 = (block_in_problem * NW + wave) * R;
  const bool active = row0 < N;
  const int64_t row_bytes = T::byte_off(K);
  const unsigned char* wbase =
      static_cast<const unsigned char*>(prob.w) + static_cast<int64_t>(active ? row0 : 0) * row_bytes;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

  typename W::Batch wa, wb;
  for (int kt = 0; kt < K; kt += KT) {
    const int kn = min(KT, K - kt);
    const int nsteps = (kn + T::kStep - 1) / T::kStep;
    // request the first batch of weights, then stage x: the two latencies overlap
    if (active) W::load_batch(wa, wbase, row_bytes, kt, kn, 0, lane, prob, row0, K);
    if (kt > 0) __syncthreads();
    if constexpr (LN) {
      // the launcher guarantees KT >= K here: the whole row is normalised at once
#pragma unroll 1
      for (int m = 0; m < M; ++m) ln_prologue_row<NW>(args.ln, prob.mu, K, m, xs + m * KT, sbuf, red, blockIdx.x == 0);
    } else {
      for (int i = threadIdx.x * 8; i < M * kn; i += NW * 64 * 8) {
        const int m = i / kn;
        const int kk = i - m * kn;
        *reinterpret_cast<uint4_t*>(xs + m * KT + kk) =
            *reinterpret_cast<const uint4_t*>(prob.x + static_cast<int64_t>(m) * K + kt + kk);
      }
    }
    __syncthreads();
    if (active) {
      // ping-pong over batches of U steps
      for (int s0 = 0; s0 < nsteps; s0 += 2 * U) {
        if (s0 + U < nsteps) W::load_batch(wb, wbase, row_bytes, kt, kn, s0 + U, lane, prob, row0, K);
        W::compute_batch(acc, wa, xs, KT, kn, s0, lane);
        if (s0 + U < nsteps) {
          if (s0 + 2 * U < nsteps) W::load_batch(wa, wbase, row_bytes, kt, kn, s0 + 2 * U, lane, prob, row0, K);
          W::compute_batch(acc, wb, xs, KT, kn, s0 + U, lane);
        }
      }
    }
  }
  if (!active) return;

#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_dpp(acc[r][m]);

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

// grid = total blocks over all problems (each block: 4 waves x R rows); dynamic LDS = M*KT*2 bytes (+ K*4 with the
// LayerNorm prologue, a separate instantiation so that launches without it keep their register budget).
template <int M, int R, int U, bool LN, int NW>
__global__ __launch_bounds__(NW * 64) void linear_gemv_kernel(LinearArgs args) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ float red[16];
  half_t* xs = reinterpret_cast<half_t*>(lds_raw);
  float* sbuf = reinterpret_cast<float*>(lds_raw + static_cast<size_t>(M) * args.KT * sizeof(half_t));
  if (blockIdx.x == 0 && args.copy.n > 0) {
    for (int i = threadIdx.x * 8; i < args.copy.n; i += NW * 64 * 8)
      *reinterpret_cast<uint4_t*>(args.copy.dst + i) = *reinterpret_cast<const uint4_t*>(args.copy.src + i);
  }
  int pi = 0;
  int first = 0;
  for (int i = 0; i < args.n_problems - 1; ++i) {
    if (static_cast<int>(blockIdx.x) >= args.block_end[i]) {
      pi = i + 1;
      first = args.block_end[i];
    }
  }
  const LinearProblem prob = args.p[pi];
  const int blk = blockIdx.x - first;
  switch (prob.fmt) {  // uniform per block
    case RWKV_FMT_W8: gemv_block<RWKV_FMT_W8, M, R, U, LN, NW>(args, prob, blk, xs, sbuf, red); break;
    case RWKV_FMT_W4: gemv_block<RWKV_FMT_W4, M, R, U, LN, NW>(args, prob, blk, xs, sbuf, red); break;
    default: gemv_block<RWKV_FMT_F16, M, R, U, LN, NW>(args, prob, blk, xs, sbuf, red); break;
  }
}

template <int M, int R, int U>
static int launch_one(hipStream_t st, LinearArgs& args) {
  const bool ln = args.ln.mode != 0;
  const int nw = 4;
  int total = 0;
  for (int i = 0; i < args.n_problems; ++i) {
    total += ceil_div(args.p[i].N, nw * R);
    args.block_end[i] = total;
  }
  size_t lds = static_cast<size_t>(M) * args.KT * sizeof(half_t);
  if (ln) lds += static_cast<size_t>(args.K) * sizeof(float);
  if (ln) {
    hipLaunchKernelGGL((linear_gemv_kernel<M, R, U, true, 4>), dim3(total), dim3(256), lds, st, args);
  } else {
    hipLaunchKernelGGL((linear_gemv_kernel<M, R, U, false, 4>), dim3(total), dim3(256), lds, st, args);
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// ---- one row (M == 1): whole weight rows in flight ---------------------------------------------------------------
// A decode step of one sequence is a chain of dependent launches, each of which moves 17-67 MB: what a launch costs
// beyond its bytes is the trip to memory at its start and the one at its end.  Here a wavefront requests ALL the
// 16-byte vectors of its rows (R = 2 rows of int8 / int4 codes, one row of fp16) in one go - K <= 4096 int8 codes
// are 4 vectors per lane and row - so every byte of the matrix is requested by the first instructions of its block
// and nothing is requested late.  With the LayerNorm prologue (LN) the block computes its own copy of
// LayerNorm(x + residual) + token-shift lerp into LDS (same formulas and rounding points as ln_fused_kernel,
// fused_ops.hip; eight or sixteen values per thread, so the sums associate differently and the last bits may
// differ from that kernel's): the stand-alone LayerNorm launch and its kernel boundary disappear.  Every block of the launch
// is resident at once (two 1024-thread blocks per CU: at most 64 registers per thread, checked at build time).
// Accumulation order per lane is that of linear_gemv_kernel (steps in order, then the same butterfly): same bits.
template <int FMT, int KCAP>
struct Row1Cfg {
  static constexpr int kRows = FMT == RWKV_FMT_F16 ? 1 : 2;
  static constexpr int kSteps = KCAP / FmtTraits<FMT>::kStep > 0 ? KCAP / FmtTraits<FMT>::kStep : 1;
};

// LayerNorm(x + res) (or of a gathered table row) + lerp against the previous token's LN output into xs[0..K), by
// the first half (int4 weights: quarter) of the block's wavefronts while the others are already waiting for their
// weights (gemv_row1_block); block 0 also stores the residual sum and the LN output.  In two parts: everything
// the prologue reads from memory is requested at once (ln_row1_request8), the arithmetic (ln_row1_finish8) reads
// no memory.  Everything that arrived goes to LDS at once (stash: NT * 4 floats for the row sum, then 4 x NT * 4
// fp16 values: LN weight, bias, previous LN output, lerp coefficients) and is read back piece by piece, each
// thread only what it wrote, so the prologue's registers stay few.
template <int V8, int M>
struct LnRow1xV {  // V8 groups of eight values, M rows
  half8_t xv[M][V8], rv[M][V8], pv[M][V8];  // per row: x, the residual, the previous token's LN output
  half8_t wv[V8], bv[V8], mv[V8];           // shared by the rows: LN weight and bias, lerp coefficients
};

// thread t of the computing wavefronts owns the groups t, t + NTL, ... (NTL computing threads).  Every row's
// operands are requested in one go, so that the rows share one trip to memory.
template <int V8, int NTL, int M>
__device__ __forceinline__ LnRow1xV<V8, M> ln_row1_request8(const LnPrologue& ln, const half_t* __restrict__ mu, int K) {
  LnRow1xV<V8, M> q;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    const int cc = c < K ? c : 0;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int64_t row = static_cast<int64_t>(m) * K;
      const int64_t xsrc = ln.mode == 2 ? ln.tokens[m] * static_cast<int64_t>(K) : row;
      q.xv[m][g] = *reinterpret_cast<const half8_t*>(ln.x + xsrc + cc);
      q.rv[m][g] = *reinterpret_cast<const half8_t*>(ln.mode == 1 ? ln.res + row + cc : ln.x + xsrc + cc);
    }
    q.wv[g] = *reinterpret_cast<const half8_t*>(ln.w + cc);
    q.bv[g] = *reinterpret_cast<const half8_t*>(ln.b + cc);
#pragma unroll
    for (int m = 0; m < M; ++m) q.pv[m][g] = *reinterpret_cast<const half8_t*>(ln.shift + static_cast<int64_t>(m) * K + cc);
    q.mv[g] = *reinterpret_cast<const half8_t*>(mu + cc);
  }
  return q;
}

#ifndef RWKV_LN_FLAGS
#define RWKV_LN_FLAGS 1
#endif

// Counters in LDS by which the wavefronts of a prologue block meet without s_barrier: a barrier counts every
// wavefront of the block, and the ones that are not computing the prologue reach it only when the memory pipeline
// has taken all their weight requests - microseconds into a large launch.  [2m], [2m + 1]: the computing wavefronts
// that have delivered their partial sum / sum of squares of row m; [kLnFlagX]: those whose part of x is in LDS.
// Zeroed by the block's first threads before the one barrier every wavefront passes on entry.
constexpr int kLnFlagX = 4;  // (up to two rows with the prologue)
struct LnFlags {
  unsigned count[kLnFlagX + 1];
};

// waits (bounded: no wavefront may spin for ever whatever happens to the others) until `n` wavefronts have arrived
__device__ __forceinline__ void ln_flag_wait(unsigned* count, unsigned n) {
  int spins = 0;
  while (__hip_atomic_load(count, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < n && ++spins < (1 << 22))
    __builtin_amdgcn_s_sleep(1);
}

__device__ __forceinline__ void ln_flag_arrive(unsigned* count) {
  if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// sum over the first NWL wavefronts of the block (the callers).  With FLAGS they meet at the counter; without, at a
// barrier that the other wavefronts pass too.
template <int NWL, bool FLAGS>
__device__ __forceinline__ float front_waves_sum(float v, int wave, float* scratch, unsigned* count) {
  v = wave_sum_uniform(v);
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  if constexpr (FLAGS) {
    ln_flag_arrive(count);
    ln_flag_wait(count, NWL);
  } else {
    __syncthreads();
  }
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < NWL; ++i) t += scratch[i];
  return t;
}

// (W4: xs in nibble-pair order, the slice sums to xsum - see w4_pair_order)
template <int NT, int V8, int NTL, int M, bool W4, bool FLAGS>
__device__ __forceinline__ void ln_row1_finish8(const LnRow1xV<V8, M>& q, const LnPrologue& ln, int K, int m, half_t* xs,
                                                float* xsum, float* stash, float* red, LnFlags* flags, bool store,
                                                int wave) {
  const int64_t row = static_cast<int64_t>(m) * K;
  constexpr int NWL = NTL / 64;  // wavefronts that compute
  half_t* hstash = reinterpret_cast<half_t*>(stash + NT * 4);
  float sum = 0.0f;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    float v[8];
    if (ln.mode == 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = h2f(q.xv[m][g][e]) + h2f(q.rv[m][g][e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = h2f(q.xv[m][g][e]);
    }
    if (c < K) sum += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    *reinterpret_cast<float4_t*>(stash + c) = float4_t{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4_t*>(stash + c + 4) = float4_t{v[4], v[5], v[6], v[7]};
    *reinterpret_cast<half8_t*>(hstash + c) = q.wv[g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 4) = q.bv[g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 8) = q.pv[m][g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 12) = q.mv[g];
  }
  __builtin_amdgcn_sched_barrier(0);
  sum = front_waves_sum<NWL, FLAGS>(sum, wave, red, &flags->count[2 * m]);
  const float mean = sum / static_cast<float>(K);
  float sv = 0.0f;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    if (c < K) {
      const float4_t v0 = *reinterpret_cast<const float4_t*>(stash + c);
      const float4_t v1 = *reinterpret_cast<const float4_t*>(stash + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = v0[e] - mean;
        sv = fmaf(d, d, sv);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = v1[e] - mean;
        sv = fmaf(d, d, sv);
      }
    }
  }
  sv = front_waves_sum<NWL, FLAGS>(sv, wave, red + NT / 64, &flags->count[2 * m + 1]);
  const float rstd = rsqrtf(sv / static_cast<float>(K) + ln.eps);
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    half8_t ov;
#pragma unroll
    for (int e = 0; e < 8; ++e) ov[e] = static_cast<half_t>(0.0f);
    if (c < K) {
      const float4_t v0 = *reinterpret_cast<const float4_t*>(stash + c);
      const float4_t v1 = *reinterpret_cast<const float4_t*>(stash + c + 4);
      const half8_t wv = *reinterpret_cast<const half8_t*>(hstash + c);
      const half8_t bv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 4);
      const half8_t pv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 8);
      const half8_t mv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 12);
      half8_t yv, xo;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float ve = e < 4 ? v0[e & 3] : v1[e & 3];
        yv[e] = f2h(fmaf((ve - mean) * rstd, h2f(wv[e]), h2f(bv[e])));
        const float yf = h2f(yv[e]);  // the lerp reads the fp16-rounded LN output
        ov[e] = f2h(fmaf(h2f(pv[e]) - yf, h2f(mv[e]), yf));
        xo[e] = f2h(ve);
      }
      if (store) {
        *reinterpret_cast<half8_t*>(ln.ln_out + row + c) = yv;
        if (ln.x_out) *reinterpret_cast<half8_t*>(ln.x_out + row + c) = xo;
      }
    }
    // zeros beyond K: the lanes past the end of a row multiply by them
    if constexpr (W4) {
      const uint4_t raw = __builtin_bit_cast(uint4_t, ov);
      const float s32 = w4_slice_sum(raw);
      *reinterpret_cast<uint4_t*>(xs + c) = w4_pair_order(raw);
      if ((threadIdx.x & 3) == 0) xsum[c >> 5] = s32;
    } else {
      *reinterpret_cast<half8_t*>(xs + c) = ov;
    }
  }
}

// The prologue of a one-row launch, kept as its own set of functions beside the several-row ones above (same
// arithmetic): written through the several-row form with M = 1, the int4 kernel came out four registers heavier -
// past the 64 that let two 1024-thread blocks share a CU - and spilled.
template <int V8>
struct LnRowOne {  // V8 groups of eight values
  half8_t xv[V8], rv[V8], wv[V8], bv[V8], pv[V8], mv[V8];
};

// thread t of the computing wavefronts owns the groups t, t + NTL, ... (NTL computing threads)
template <int V8, int NTL>
__device__ __forceinline__ LnRowOne<V8> ln_one_request8(const LnPrologue& ln, const half_t* __restrict__ mu, int K) {
  const int64_t xsrc = ln.mode == 2 ? ln.tokens[0] * static_cast<int64_t>(K) : 0;
  LnRowOne<V8> q;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    const int cc = c < K ? c : 0;
    q.xv[g] = *reinterpret_cast<const half8_t*>(ln.x + xsrc + cc);
    q.rv[g] = *reinterpret_cast<const half8_t*>(ln.mode == 1 ? ln.res + cc : ln.x + xsrc + cc);
    q.wv[g] = *reinterpret_cast<const half8_t*>(ln.w + cc);
    q.bv[g] = *reinterpret_cast<const half8_t*>(ln.b + cc);
    q.pv[g] = *reinterpret_cast<const half8_t*>(ln.shift + cc);
    q.mv[g] = *reinterpret_cast<const half8_t*>(mu + cc);
  }
  return q;
}

// sum over the first NWL wavefronts of the block (the callers).  With FLAGS they meet at the counter; without, at a
// barrier that the other wavefronts pass too.
template <int NWL, bool FLAGS>
__device__ __forceinline__ float front_waves_sum_one(float v, int wave, float* scratch, unsigned* count) {
  v = wave_sum_uniform(v);
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  if constexpr (FLAGS) {
    ln_flag_arrive(count);
    ln_flag_wait(count, NWL);
  } else {
    __syncthreads();
  }
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < NWL; ++i) t += scratch[i];
  return t;
}

template <int NT, int V8, int NTL, bool W4, bool FLAGS>
__device__ __forceinline__ void ln_one_finish8(const LnRowOne<V8>& q, const LnPrologue& ln, int K, half_t* xs,
                                                float* xsum, float* stash, float* red, LnFlags* flags, bool store,
                                                int wave) {
  constexpr int NWL = NTL / 64;  // wavefronts that compute
  half_t* hstash = reinterpret_cast<half_t*>(stash + NT * 4);
  float sum = 0.0f;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    float v[8];
    if (ln.mode == 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = h2f(q.xv[g][e]) + h2f(q.rv[g][e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = h2f(q.xv[g][e]);
    }
    if (c < K) sum += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    *reinterpret_cast<float4_t*>(stash + c) = float4_t{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4_t*>(stash + c + 4) = float4_t{v[4], v[5], v[6], v[7]};
    *reinterpret_cast<half8_t*>(hstash + c) = q.wv[g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 4) = q.bv[g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 8) = q.pv[g];
    *reinterpret_cast<half8_t*>(hstash + c + NT * 12) = q.mv[g];
  }
  __builtin_amdgcn_sched_barrier(0);
  sum = front_waves_sum_one<NWL, FLAGS>(sum, wave, red, &flags->count[0]);
  const float mean = sum / static_cast<float>(K);
  float sv = 0.0f;
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    if (c < K) {
      const float4_t v0 = *reinterpret_cast<const float4_t*>(stash + c);
      const float4_t v1 = *reinterpret_cast<const float4_t*>(stash + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = v0[e] - mean;
        sv = fmaf(d, d, sv);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = v1[e] - mean;
        sv = fmaf(d, d, sv);
      }
    }
  }
  sv = front_waves_sum_one<NWL, FLAGS>(sv, wave, red + NT / 64, &flags->count[1]);
  const float rstd = rsqrtf(sv / static_cast<float>(K) + ln.eps);
#pragma unroll
  for (int g = 0; g < V8; ++g) {
    const int c = (threadIdx.x + g * NTL) * 8;
    half8_t ov;
#pragma unroll
    for (int e = 0; e < 8; ++e) ov[e] = static_cast<half_t>(0.0f);
    if (c < K) {
      const float4_t v0 = *reinterpret_cast<const float4_t*>(stash + c);
      const float4_t v1 = *reinterpret_cast<const float4_t*>(stash + c + 4);
      const half8_t wv = *reinterpret_cast<const half8_t*>(hstash + c);
      const half8_t bv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 4);
      const half8_t pv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 8);
      const half8_t mv = *reinterpret_cast<const half8_t*>(hstash + c + NT * 12);
      half8_t yv, xo;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float ve = e < 4 ? v0[e & 3] : v1[e & 3];
        yv[e] = f2h(fmaf((ve - mean) * rstd, h2f(wv[e]), h2f(bv[e])));
        const float yf = h2f(yv[e]);  // the lerp reads the fp16-rounded LN output
        ov[e] = f2h(fmaf(h2f(pv[e]) - yf, h2f(mv[e]), yf));
        xo[e] = f2h(ve);
      }
      if (store) {
        *reinterpret_cast<half8_t*>(ln.ln_out + c) = yv;
        if (ln.x_out) *reinterpret_cast<half8_t*>(ln.x_out + c) = xo;
      }
    }
    // zeros beyond K: the lanes past the end of a row multiply by them
    if constexpr (W4) {
      const uint4_t raw = __builtin_bit_cast(uint4_t, ov);
      const float s32 = w4_slice_sum(raw);
      *reinterpret_cast<uint4_t*>(xs + c) = w4_pair_order(raw);
      if ((threadIdx.x & 3) == 0) xsum[c >> 5] = s32;
    } else {
      *reinterpret_cast<half8_t*>(xs + c) = ov;
    }
  }
}

// One block.  A wavefront cannot do both at once: it stalls on its weight requests until the memory pipeline has
// room for them - late in a 67 MB launch that takes microseconds (timestamps: the last wavefronts get their
// requests out 11 us after the launch began) - and a prologue behind the requests would end up at the tail of the
// launch, while a prologue before them leaves HBM idle for its 1.5 us.  So the wavefronts share the work: some
// compute the prologue and request their weights afterwards, the others request theirs at once and meet the first
// at the barrier (7.2B shape, int8: 1.79 -> 1.72 ms per step against the prologue in every wavefront first).
template <int FMT, int NT, bool LN, int M, int RX>
__device__ __forceinline__ void gemv_row1_block(const LinearArgs& args, const LinearProblem& prob, int blk, half_t* xs,
                                               float* red, LnFlags* flags) {
  using T = FmtTraits<FMT>;
  constexpr int KCAP = LN ? NT * 4 : NT * 8;  // values of x the block stages per row: one slice per thread
  using Cfg = Row1Cfg<FMT, KCAP>;
  constexpr int R = Cfg::kRows * RX;
  constexpr int S = Cfg::kSteps;
  constexpr int NW = NT / 64;
  const int K = args.K;
  const int N = prob.N;
  // wavefront-uniform values in scalar registers: row addresses then cost no vector registers
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int row0 = (blk * NW + wave) * R;
  const bool active = row0 < N;
  const int64_t row_bytes = T::byte_off(K);
  const unsigned char* wbase = static_cast<const unsigned char*>(prob.w) + static_cast<int64_t>(active ? row0 : 0) * row_bytes;

  // With the prologue: the first half of the wavefronts computes it (eight values per thread) and requests its
  // weights afterwards; the second half requests its weights at once, so that HBM streams while the prologue runs.
  // (half of them for int8 and fp16 weights; a quarter for int4, whose wavefronts have three requests per vector
  // to get out: 7.2B shape, ms per step with a half / a quarter: int8 1.72 / 1.75, int4 1.70 / 1.64)
  constexpr bool kW4 = FMT == RWKV_FMT_W4;
  // LDS: M rows of x, then (used by int4 blocks) the sums of every 32 values of each row, then the prologue's stash
  float* xsum = reinterpret_cast<float*>(xs + M * KCAP);
  float* stash = xsum + M * (KCAP / 32);
  constexpr int NTL = NT / (FMT == RWKV_FMT_W4 ? 4 : 2);  // threads that compute the prologue
  constexpr int V8 = NT * 4 / (NTL * 8);  // groups of eight values per computing thread
  const bool ln_wave = LN && wave < NTL / 64;
  uint4_t xq[M];
#pragma unroll
  for (int m = 0; m < M; ++m) xq[m] = uint4_t{0u, 0u, 0u, 0u};
  if constexpr (LN) {
    // (below, after the row scales)
  } else if (prob.x_f32 != nullptr) {
    // x = f16(x_f32 * gate): the products are formed here, one rounding each
    if (static_cast<int>(threadIdx.x) * 8 < K) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float* xf = prob.x_f32 + static_cast<int64_t>(m) * K + threadIdx.x * 8;
        const float4_t f0 = *reinterpret_cast<const float4_t*>(xf);
        const float4_t f1 = *reinterpret_cast<const float4_t*>(xf + 4);
        const half8_t gq = *reinterpret_cast<const half8_t*>(prob.x_gate + static_cast<int64_t>(m) * K + threadIdx.x * 8);
        half8_t xh;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          xh[e] = f2h(f0[e] * h2f(gq[e]));
          xh[4 + e] = f2h(f1[e] * h2f(gq[4 + e]));
        }
        xq[m] = __builtin_bit_cast(uint4_t, xh);
      }
    }
  } else {
    if (static_cast<int>(threadIdx.x) * 8 < K) {
#pragma unroll
      for (int m = 0; m < M; ++m)
        xq[m] = *reinterpret_cast<const uint4_t*>(prob.x + static_cast<int64_t>(m) * K + threadIdx.x * 8);
    }
  }
  half_t row_scale[R];
#pragma unroll
  for (int r = 0; r < R; ++r) row_scale[r] = static_cast<half_t>(1.0f);
  // the compiler must not move the reads of x behind the weight reads below (loads complete in issue order)
  __builtin_amdgcn_sched_barrier(0);

  // No load sits under a branch: a lane past the end of the row re-reads the row's last vector (and multiplies it
  // by the zeros that pad x).
  uint4_t w[S][R];
  half_t sc[S][R];
  uint8_t zp[S][R];
  auto request = [&](int st) {
    const int k0 = st * T::kStep + lane * T::kElems;
    const int kc = k0 < K ? k0 : K - T::kElems;
#pragma unroll
    for (int r = 0; r < R; ++r)
      w[st][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(wbase + r * row_bytes + T::byte_off(kc)));
  };
  // int4: every group's scale and zero point, requested before any codes.  Loads return in issue order: were these
  // issued among the codes (where the compiler would put them), the first product would wait for the last codes,
  // and the whole dot phase - a few microseconds of VALU work on a launch of this size - would start only when the
  // stream from HBM has ended, instead of running under it.
  auto request_all = [&]() {
    // the int8 rows' output scales too, ahead of the codes: read at the end they would cost every wavefront one
    // more trip to memory (and before the prologue, its wavefronts would sit out that trip before their own reads)
    if constexpr (FMT == RWKV_FMT_W8) {
#pragma unroll
      for (int r = 0; r < R; ++r) row_scale[r] = prob.scale[active ? row0 + r : r];
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (FMT == RWKV_FMT_W4) {
#pragma unroll
      for (int st = 0; st < S; ++st) {
        const int k0 = st * T::kStep + lane * T::kElems;
        const int kc = k0 < K ? k0 : K - T::kElems;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int64_t gi = static_cast<int64_t>(active ? row0 + r : r) * (K >> 7) + (kc >> 7);
          sc[st][r] = prob.scale[gi];
          zp[st][r] = prob.zp[gi];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int st = 0; st < S; ++st) request(st);
  };
  // The products, once x is in LDS.  per (row of W, row of x): steps in order, the lane's pairs in order - the order
  // of one-row launches, same bits
  auto dots = [&]() {
    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;
#pragma unroll
    for (int st = 0; st < S; ++st) {
      const int k0 = st * T::kStep + lane * T::kElems;
      if (st * T::kStep < K && k0 + T::kElems <= KCAP) {  // (the second test only where a step is wider than KCAP)
        constexpr int XV = T::kElems / 2;
#pragma unroll
        for (int m = 0; m < M; ++m) {
          half2_t xv[XV];
#pragma unroll
          for (int q = 0; q < XV / 4; ++q) {
            const uint4_t t = *reinterpret_cast<const uint4_t*>(xs + m * KCAP + k0 + q * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) xv[q * 4 + e] = as_half2(t[e]);
          }
          if constexpr (kW4) {
            // xv is in nibble-pair order already; the slice's sum takes out the offset of 16 and the zero point
            const float xs32 = xsum[m * (KCAP / 32) + (k0 >> 5)];
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const float part = w4_dot_offset16(w[st][r], xv, 0.0f);
              const float off = -(16.0f + static_cast<float>(zp[st][r]));
              acc[r][m] = fmaf(fmaf(off, xs32, part), h2f(sc[st][r]), acc[r][m]);
              // one vector's arithmetic stays together, in the order the vectors were requested
              __builtin_amdgcn_sched_barrier(0);
            }
          } else {
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r][m] = WeightVec<FMT>::dot(w[st][r], xv, acc[r][m]);
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = wave_sum_dpp(acc[r][m]);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = row0 + r;
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float v = round_h(acc[r][m] * h2f(row_scale[r]));
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
  };
  // x in LDS: one slice per thread and row (rows KCAP values apart), zeros beyond K
  if constexpr (LN) {
    // two code paths, so that the prologue's operands and the weight vectors never hold registers together; the
    // second path passes the two barriers of the first one's block sums, once per row
    constexpr bool kFlags = RWKV_LN_FLAGS != 0;
    constexpr unsigned NWL = NTL / 64;
    if (ln_wave) {
      if constexpr (M == 1) {
        const LnRowOne<V8> lnq = ln_one_request8<V8, NTL>(args.ln, prob.mu, K);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kFlags) {
          // the prologue's operands are in the memory pipeline ahead of any weights of this block
          if (threadIdx.x <= kLnFlagX) flags->count[threadIdx.x] = 0u;
          __syncthreads();
          // (nothing that waits for the operands may move above the barrier: the other wavefronts wait there)
          __builtin_amdgcn_sched_barrier(0);
        }
        ln_one_finish8<NT, V8, NTL, kW4, kFlags>(lnq, args.ln, K, xs, xsum, stash, red, flags, blockIdx.x == 0, wave);
        __builtin_amdgcn_sched_barrier(0);
      } else {
        const LnRow1xV<V8, M> lnq = ln_row1_request8<V8, NTL, M>(args.ln, prob.mu, K);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (kFlags) {
          if (threadIdx.x <= kLnFlagX) flags->count[threadIdx.x] = 0u;
          __syncthreads();
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int m = 0; m < M; ++m) {
          // (the stash of row m is rewritten by row m + 1 only after every wavefront has passed row m's second
          // meeting, i.e. has read what it needs of it: each thread reads only what it wrote)
          ln_row1_finish8<NT, V8, NTL, M, kW4, kFlags>(lnq, args.ln, K, m, xs + m * KCAP, xsum + m * (KCAP / 32), stash,
                                                       red, flags, blockIdx.x == 0, wave);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if constexpr (kFlags) ln_flag_arrive(&flags->count[kLnFlagX]);
      request_all();
      // Each path has its own copy of the products.  Where the two paths met before them, the compiler's wait for
      // the first vector became a wait for one of the last (it merges the two paths' lists of loads in flight
      // conservatively), and the arithmetic - microseconds of it per launch - ran after the stream, not under it.
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kFlags) {
        ln_flag_wait(&flags->count[kLnFlagX], NWL);
      } else {
        __syncthreads();
      }
      if (active) dots();
      return;
    } else {
      if constexpr (kFlags) __syncthreads();
      request_all();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kFlags) {
        ln_flag_wait(&flags->count[kLnFlagX], NWL);
      } else {
#pragma unroll 1
        for (int m = 0; m < M; ++m) {
          __syncthreads();
          __syncthreads();
        }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
      }
      if (active) dots();
      return;
    }
  } else {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      if constexpr (kW4) {
        const float s32 = w4_slice_sum(xq[m]);
        *reinterpret_cast<uint4_t*>(xs + m * KCAP + threadIdx.x * 8) = w4_pair_order(xq[m]);
        if ((threadIdx.x & 3) == 0) xsum[m * (KCAP / 32) + (threadIdx.x >> 2)] = s32;
      } else {
        *reinterpret_cast<uint4_t*>(xs + m * KCAP + threadIdx.x * 8) = xq[m];
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    request_all();
  }
  __builtin_amdgcn_sched_barrier(0);
  __syncthreads();
  if (!active) return;
  dots();
}

// grid = blocks over all problems; a block of NT threads covers NT/64 * (1 or 2) rows of W for all M rows of x; dynamic
// LDS = M rows of x (NT * 4 fp16 values each with the prologue, NT * 8 without) + the prologue's stash.  DF is the
// format of the launch's quantised problems; fp16 problems (the LoRA rank-ins) may ride along.
// With the prologue and 1024 threads two blocks must share a CU (every block of the launch resident at once): 8
// wavefronts per SIMD, i.e. at most 64 registers - asked for here, and checked from the compiler's resource report at
// build time.  (Two rows of int4 codes do not fit that budget and run one block per CU.)
template <int NT, bool LN, int DF, int M, int RX>
__global__ __launch_bounds__(NT, (LN && NT == 1024 && (M == 1 || DF != RWKV_FMT_W4)) ? 8 / RX : (LN && NT == 1024 ? 4 : 1))
void linear_gemv_row1_kernel(LinearArgs args) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ float red[2 * (NT / 64)];
  __shared__ LnFlags flags;
  half_t* xs = reinterpret_cast<half_t*>(lds_raw);
  if (blockIdx.x == 0 && args.copy.n > 0) {
    for (int i = threadIdx.x * 8; i < args.copy.n; i += NT * 8)
      *reinterpret_cast<uint4_t*>(args.copy.dst + i) = *reinterpret_cast<const uint4_t*>(args.copy.src + i);
  }
  int pi = 0;
  int first = 0;
  for (int i = 0; i < args.n_problems - 1; ++i) {
    if (static_cast<int>(blockIdx.x) >= args.block_end[i]) {
      pi = i + 1;
      first = args.block_end[i];
    }
  }
  const LinearProblem prob = args.p[pi];
  const int blk = blockIdx.x - first;
  if (DF != RWKV_FMT_F16 && prob.fmt == DF) {  // uniform per block
    gemv_row1_block<DF, NT, LN, M, RX>(args, prob, blk, xs, red, &flags);
  } else {
    gemv_row1_block<RWKV_FMT_F16, NT, LN, M, RX>(args, prob, blk, xs, red, &flags);
  }
}

// The quantised format of the launch (fp16 if none), or -1 if the launch mixes int8 and int4 problems or a row is
// longer than a wavefront holds in registers (K > 4096).
static int row1_format(const LinearArgs& args) {
  if (args.K > 4096) return -1;
  int df = RWKV_FMT_F16;
  for (int i = 0; i < args.n_problems; ++i) {
    const int fmt = args.p[i].fmt;
    if (fmt == RWKV_FMT_F16) continue;
    if (df != RWKV_FMT_F16 && df != fmt) return -1;
    df = fmt;
  }
  return df;
}

// Rows of x the whole-rows-in-flight kernel takes: up to 4 (each more row costs every weight vector another eight
// v_dot2 and two LDS reads; beyond 4 the matrix core is the better tool), up to 2 with the LayerNorm prologue (each
// row's prologue runs before the computing wavefronts request their weights, and the stash shares the LDS).
constexpr int kRow1MaxRows = 4;
constexpr int kRow1MaxRowsLn = 2;
static_assert(2 * kRow1MaxRowsLn <= kLnFlagX, "two counters per prologue row");

template <int NT, bool LN, int DF, int M, int RX = 1>
static int launch_row1(hipStream_t st, LinearArgs& args) {
  int total = 0;
  for (int i = 0; i < args.n_problems; ++i) {
    const int rows_per_block = (NT / 64) * (args.p[i].fmt == RWKV_FMT_F16 ? 1 : 2) * RX;
    total += ceil_div(args.p[i].N, rows_per_block);
    args.block_end[i] = total;
  }
  // int4 codes, rows of 4096: a launch with more blocks than CUs doubles the rows per wavefront, so that one block
  // per CU covers it (one prologue per CU instead of two, whose second one has its operands queued behind the first
  // block's weights; the short int4 stream cannot hide that: 7.2B shape, 1.56 -> 1.48 ms per step).  The int8
  // stream is long enough to hide it and runs a little better with two blocks per CU (1.70 against 1.73 ms).
  if constexpr (RX == 1 && LN && NT == 1024 && DF == RWKV_FMT_W4) {
    if (total > device_cu_count()) return launch_row1<NT, LN, DF, M, 2>(st, args);
  }
  args.KT = LN ? NT * 4 : NT * 8;
  // x rows, the slice sums of int4 blocks (4 bytes per 32 values and row), with the prologue also its stash
  const size_t lds = static_cast<size_t>(args.KT) * (2 * M + (LN ? 4 + 4 * 2 : 0)) + static_cast<size_t>(M) * (args.KT / 32) * 4;
  if (lds > 48 * 1024) {  // beyond the default limit of dynamic LDS: raised once per instantiation
    static bool raised = false;
    if (!raised) {
      RWKV_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_gemv_row1_kernel<NT, LN, DF, M, RX>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
      raised = true;
    }
  }
  hipLaunchKernelGGL((linear_gemv_row1_kernel<NT, LN, DF, M, RX>), dim3(total), dim3(NT), lds, st, args);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

template <int NT, bool LN, int M>
static int launch_row1_fmt(hipStream_t st, LinearArgs& args, int df) {
  switch (df) {
    case RWKV_FMT_W8: return launch_row1<NT, LN, RWKV_FMT_W8, M>(st, args);
    case RWKV_FMT_W4: return launch_row1<NT, LN, RWKV_FMT_W4, M>(st, args);
    default: return launch_row1<NT, LN, RWKV_FMT_F16, M>(st, args);
  }
}

// Block size by row length: one slice of x per thread (4 values with the prologue, 8 without).
template <int M>
static int launch_row1_any(hipStream_t st, LinearArgs& args, int df) {
  const int K = args.K;
  if constexpr (M <= kRow1MaxRowsLn) {
    if (args.ln.mode != 0) {
      if (K <= 1024) return launch_row1_fmt<256, true, M>(st, args, df);
      if (K <= 2048) return launch_row1_fmt<512, true, M>(st, args, df);
      return launch_row1_fmt<1024, true, M>(st, args, df);
    }
  }
  if (K <= 2048) return launch_row1_fmt<256, false, M>(st, args, df);
  return launch_row1_fmt<512, false, M>(st, args, df);
}


// ---- 5..16 rows: the same stream of whole rows, the products on the matrix core --------------------------------------
// From five rows on, the GEMV's per-row VALU work (one v_dot2 per row and pair of weights) costs more than the stream
// it runs under.  Here v_mfma_f32_16x16x32_f16 takes the rows of x as the sixteen columns of its B operand: a
// wavefront owns sixteen rows of W and a part of K - lane (r, q) = (lane % 16, lane / 16) requests, per step, the
// 16 bytes of row r that follow the 16 bytes of lane (r, q - 1), so a step covers 64 bytes of each of the sixteen
// rows - and has up to 16 vectors in flight at once (K = 4096 int8 codes in 4 parts: all of them), as the GEMV's
// wavefronts have theirs.  A block of 16 wavefronts is G groups of sixteen rows x 16 / G parts of K (G = 4 where
// that still gives every CU a block, else 1); the parts' 16 x 16 partial products meet in LDS and are added in part
// order.  x (M rows, fp16) is staged in LDS once per block, rows K + 8 values apart (the sixteen lanes of a b128
// read then hit different banks); lanes whose column is no row of x read row 0 and their products are dropped.
// int8 codes become fp16 (exact) on the way, the row scale multiplies the sum.
//
// The wavefronts share the start of the launch like those of the GEMV with the LayerNorm prologue: the first half
// brings x into LDS (8 or, for 9..16 rows of 4096 values, 16 vectors per thread) and requests its weights
// afterwards, the second half requests its weights at once; they meet at a counter in LDS, not at a barrier - a
// barrier counts every wavefront, and a wavefront reaches it only when the memory pipeline has taken all its
// requests.
constexpr int kRowsMfmaMax = 16;
constexpr int kRowsMfmaMin = 5;
constexpr int kRowsMfmaThreads = 1024;
constexpr int kRowsMfmaXVecs = 8;  // 16-byte vectors of x per staging thread (twice as many for 9..16 rows of 4096)

// LayerNorm(x + res) (or of a gathered table row) + token-shift lerp of up to 8 rows straight into the block's LDS
// copy of x, by the staging wavefronts of a few-row matrix-core block: wavefront m owns row m (lane l the 8-value
// slices l, l + 64, ...), so a row's statistics need no other wavefront.  Same formulas and rounding points as
// ln_fused_kernel (fused_ops.hip), whose thread j * 64 + l holds this lane's slice j (one wavefront sum per j, added
// in j order); the sums inside a slice and a wavefront associate differently, so the last bits may differ from that
// kernel's.  LN weight, bias and this problem's lerp coefficients, which every row
// needs whole, are fetched once per block (thread t its slice t) and passed through LDS (hst: 3 x K values);
// block 0 of the launch also stores the residual sum and the LN output.
constexpr int kRowsMfmaLnRows = 8;
constexpr int kRowsMfmaLnSlices = 8;  // K <= 4096 = 8 x 64 lanes x 8 values

__device__ __forceinline__ void rows_mfma_ln_prologue(const LnPrologue& ln, const half_t* __restrict__ mu, int K, int M,
                                                      half_t* xs, int xstride, half_t* hst, LnFlags* flags, bool store) {
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int nj = K >> 9;             // slices per lane
  const bool row = wave < M;         // (wavefront-uniform)
  const int64_t roff = static_cast<int64_t>(wave) * K;
  // In the order of use, which is the order of arrival: the previous token's LN output (parked in the row's place in
  // xs until the lerp), the shared vectors (to hst), then x and the residual, which stay in registers.
  half8_t xv[kRowsMfmaLnSlices], rv[kRowsMfmaLnSlices];
  {
    half8_t pv[kRowsMfmaLnSlices];
    if (row) {
      const half_t* ps = ln.shift + roff + lane * 8;
#pragma unroll
      for (int j = 0; j < kRowsMfmaLnSlices; ++j)
        if (j < nj) pv[j] = *reinterpret_cast<const half8_t*>(ps + j * 512);
    }
    const int ct = static_cast<int>(threadIdx.x) * 8;  // (staging threads: 0 .. 511)
    const int cc = ct < K ? ct : 0;
    const half8_t wv = *reinterpret_cast<const half8_t*>(ln.w + cc);
    const half8_t bv = *reinterpret_cast<const half8_t*>(ln.b + cc);
    const half8_t mv = *reinterpret_cast<const half8_t*>(mu + cc);
    __builtin_amdgcn_sched_barrier(0);
    if (row) {
      const int64_t xsrc = ln.mode == 2 ? ln.tokens[wave] * static_cast<int64_t>(K) : roff;
      const half_t* px = ln.x + xsrc + lane * 8;
      const half_t* pr = ln.mode == 1 ? ln.res + roff + lane * 8 : px;
#pragma unroll
      for (int j = 0; j < kRowsMfmaLnSlices; ++j) {
        if (j < nj) {
          xv[j] = *reinterpret_cast<const half8_t*>(px + j * 512);
          rv[j] = *reinterpret_cast<const half8_t*>(pr + j * 512);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // everything the prologue reads is in the memory pipeline ahead of any weights of this block
    if (threadIdx.x <= kLnFlagX) flags->count[threadIdx.x] = 0u;
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    if (row) {
#pragma unroll
      for (int j = 0; j < kRowsMfmaLnSlices; ++j)
        if (j < nj) *reinterpret_cast<half8_t*>(xs + wave * xstride + (j * 64 + lane) * 8) = pv[j];
    }
    if (ct < K) {
      *reinterpret_cast<half8_t*>(hst + ct) = wv;
      *reinterpret_cast<half8_t*>(hst + K + ct) = bv;
      *reinterpret_cast<half8_t*>(hst + 2 * K + ct) = mv;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  ln_flag_arrive(&flags->count[0]);
  if (row) {
    // the row as fp32 sums from here on (as many registers as x and the residual took)
    float v[kRowsMfmaLnSlices][8];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kRowsMfmaLnSlices; ++j) {
      if (j < nj) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[j][e] = ln.mode == 1 ? h2f(xv[j][e]) + h2f(rv[j][e]) : h2f(xv[j][e]);
        sum += wave_sum_uniform(((v[j][0] + v[j][1]) + (v[j][2] + v[j][3])) + ((v[j][4] + v[j][5]) + (v[j][6] + v[j][7])));
        // (slice by slice: converted all at once, the fp32 sums and their fp16 sources would not fit the registers)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const float mean = sum / static_cast<float>(K);
    float sv = 0.0f;
#pragma unroll
    for (int j = 0; j < kRowsMfmaLnSlices; ++j) {
      if (j < nj) {
        float q = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float d = v[j][e] - mean;
          q = fmaf(d, d, q);
        }
        sv += wave_sum_uniform(q);
      }
    }
    const float rstd = rsqrtf(sv / static_cast<float>(K) + ln.eps);
    // (the differences from the mean are formed again below: kept from the pass above - which the compiler would do,
    // seeing the same subtraction - they would be 64 registers more than there are)
    float mean_again = mean;
    asm volatile("" : "+v"(mean_again));
    ln_flag_wait(&flags->count[0], kRowsMfmaThreads / 128);  // LN weight, bias and coefficients are in LDS
#pragma unroll
    for (int j = 0; j < kRowsMfmaLnSlices; ++j) {
      if (j < nj) {
        const int c = (j * 64 + lane) * 8;
        const half8_t w8 = *reinterpret_cast<const half8_t*>(hst + c);
        const half8_t b8 = *reinterpret_cast<const half8_t*>(hst + K + c);
        const half8_t m8 = *reinterpret_cast<const half8_t*>(hst + 2 * K + c);
        const half8_t p8 = *reinterpret_cast<const half8_t*>(xs + wave * xstride + c);  // (parked above by this lane)
        half8_t yv, ov, xo;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float ve = v[j][e];
          yv[e] = f2h(fmaf((ve - mean_again) * rstd, h2f(w8[e]), h2f(b8[e])));
          const float yf = h2f(yv[e]);  // the lerp reads the fp16-rounded LN output
          ov[e] = f2h(fmaf(h2f(p8[e]) - yf, h2f(m8[e]), yf));
          xo[e] = f2h(ve);
        }
        *reinterpret_cast<half8_t*>(xs + wave * xstride + c) = ov;
        if (store) {
          *reinterpret_cast<half8_t*>(ln.ln_out + roff + c) = yv;
          if (ln.x_out) *reinterpret_cast<half8_t*>(ln.x_out + roff + c) = xo;
        }
      }
    }
  }
}

// Groups of sixteen rows in a block of fp16 weights, by those of the launch's int8 blocks: half as many where that
// is possible, so that every block of a launch streams the same number of bytes and a wavefront's vectors of either
// format fit one batch (7.2B shape, r/k/v with the fp16 rank-ins riding along).
constexpr int rows_mfma_groups_f16(int g) { return g >= 2 ? g / 2 : g; }

template <int FMT, int NB, int G, bool LN, int XV>
__device__ __forceinline__ void rows_mfma_block(const LinearArgs& args, const LinearProblem& prob, int blk, int M,
                                                half_t* xs, int xstride, float* part, LnFlags* flags) {
  unsigned* flag = &flags->count[kLnFlagX];
  constexpr int EB = FMT == RWKV_FMT_F16 ? 2 : 1;    // bytes per weight
  constexpr int KV = 16 / EB;                         // weights per 16-byte vector
  constexpr int P = 16 / G;                           // parts of K
  const int K = args.K;
  const int N = prob.N;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int g = wave / P, kp = wave % P;
  const int r = lane & 15, kq = lane >> 4;
  const int KP = K / P;                               // this wavefront's part of K
  const int steps = KP / (4 * KV);                    // vectors per lane: a step is 4 * KV values of a row
  const int n0 = (blk * G + g) * 16;
  const bool active = n0 < N;
  const int64_t ldw = prob.ldw ? prob.ldw : K;
  const unsigned char* wrow = static_cast<const unsigned char*>(prob.w) +
                              (static_cast<int64_t>(active ? n0 + r : r) * ldw + static_cast<int64_t>(kp) * KP + kq * KV) * EB;
  const half_t* xrow = xs + (r < M ? r : 0) * xstride + kp * KP + kq * KV;
  float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
  uint4_t w[NB];
  auto request = [&](int s0) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
      w[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(wrow + static_cast<int64_t>(s0 + i) * 64));
  };
  auto products = [&](int s0) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const half_t* xp = xrow + (s0 + i) * 4 * KV;
      if constexpr (FMT == RWKV_FMT_F16) {
        const half8_t b = *reinterpret_cast<const half8_t*>(xp);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, w[i]), b, acc, 0, 0, 0);
      } else {
        half2_t c[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) cvt_i8x4(w[i][d], c[2 * d], c[2 * d + 1]);
        const half8_t a0 = {c[0][0], c[0][1], c[1][0], c[1][1], c[2][0], c[2][1], c[3][0], c[3][1]};
        const half8_t a1 = {c[4][0], c[4][1], c[5][0], c[5][1], c[6][0], c[6][1], c[7][0], c[7][1]};
        const half8_t b0 = *reinterpret_cast<const half8_t*>(xp);
        const half8_t b1 = *reinterpret_cast<const half8_t*>(xp + 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc, 0, 0, 0);
      }
    }
  };
  // x of this problem: M rows of K / 8 vectors (the rows ldx values apart)
  const int kv = K >> 3;
  const int64_t ldx = prob.ldx ? prob.ldx : K;
  constexpr int NTS = kRowsMfmaThreads / 2;  // staging threads: the first half of the wavefronts
  auto stage_x = [&]() {
    uint4_t xv[XV];
#pragma unroll
    for (int j = 0; j < XV; ++j) {
      const int i = threadIdx.x + j * NTS;
      xv[j] = uint4_t{0u, 0u, 0u, 0u};
      if (i < M * kv) {
        const int m = i / kv, c = (i - m * kv) * 8;
        xv[j] = *reinterpret_cast<const uint4_t*>(prob.x + m * ldx + c);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    // x is in the memory pipeline ahead of any weights of this block
    if (threadIdx.x <= kLnFlagX) flags->count[threadIdx.x] = 0u;
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < XV; ++j) {
      const int i = threadIdx.x + j * NTS;
      if (i < M * kv) {
        const int m = i / kv, c = (i - m * kv) * 8;
        *reinterpret_cast<uint4_t*>(xs + m * xstride + c) = xv[j];
      }
    }
  };
  constexpr unsigned NWS = NTS / 64;
  if (wave < static_cast<int>(NWS)) {
    if constexpr (LN) {
      half_t* hst = reinterpret_cast<half_t*>(part + 16 * 256);
      rows_mfma_ln_prologue(args.ln, prob.mu, K, M, xs, xstride, hst, flags, blockIdx.x == 0);
    } else {
      stage_x();
    }
    __builtin_amdgcn_sched_barrier(0);
    ln_flag_arrive(flag);
    request(0);
    __builtin_amdgcn_sched_barrier(0);
    ln_flag_wait(flag, NWS);
  } else {
    __syncthreads();
    request(0);
    __builtin_amdgcn_sched_barrier(0);
    ln_flag_wait(flag, NWS);
  }
  __builtin_amdgcn_sched_barrier(0);
  products(0);
#pragma unroll 1
  for (int s0 = NB; s0 < steps; s0 += NB) {
    request(s0);
    products(s0);
  }
  // lane (j, i4) = (lane % 16, lane / 16) holds the products of rows n0 + 4 * i4 + v (v = 0..3) of W with row j of x
#pragma unroll
  for (int v = 0; v < 4; ++v) part[wave * 256 + v * 64 + lane] = acc[v];
  __syncthreads();
  // G * 256 sums: thread t adds the parts of one (row of W, row of x), in part order
  {
    const int t = threadIdx.x;
    const int og = t >> 8, v = (t >> 6) & 3, l = t & 63;
    const int n = (blk * G + og) * 16 + 4 * (l >> 4) + v;
    const int m = l & 15;
    if (og < G && m < M && n < N) {
      const float* ps = part + og * P * 256 + v * 64 + l;
      float sum = ps[0];
#pragma unroll
      for (int q = 1; q < P; ++q) sum += ps[q * 256];
      const int64_t o = static_cast<int64_t>(m) * N + n;
      if (prob.raw_f32) {  // (uniform per block)
        static_cast<float*>(prob.y)[o] = sum;
        return;
      }
      if constexpr (FMT == RWKV_FMT_W8) sum *= h2f(prob.scale[n]);
      sum = round_h(sum);
      if (args.epilogue == RWKV_EPI_RELU_SQUARE) {
        sum = fmaxf(sum, 0.0f);
        sum = round_h(sum * sum);
      }
      if (args.out_f32) {
        static_cast<float*>(prob.y)[o] = sum;
      } else {
        static_cast<half_t*>(prob.y)[o] = f2h(sum);
      }
    }
  }
}

// grid = blocks of 16 * G rows of W over all problems, which share x (M <= 16 rows) only in shape: each problem has
// its own x.  Dynamic LDS: M rows of K + 8 fp16 values, then 16 x 256 floats of partial products, with the
// LayerNorm prologue also 3 x K fp16 values (LN weight, bias, lerp coefficients).  One block per CU
// (1024 threads, up to 128 registers).  DF: format of the quantised problems (int8); fp16 problems may ride along
// (twice the steps, in batches of the same size).
template <int DF, int NB, int G, bool LN, int XV>
__global__ __launch_bounds__(kRowsMfmaThreads)
void linear_rows_mfma_kernel(LinearArgs args, int M) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  __shared__ LnFlags flags;
  half_t* xs = reinterpret_cast<half_t*>(lds_raw);
  const int xstride = args.K + 8;
  float* part = reinterpret_cast<float*>(lds_raw + static_cast<size_t>(M) * xstride * sizeof(half_t));
  if (blockIdx.x == 0 && args.copy.n > 0) {
    for (int i = threadIdx.x * 8; i < args.copy.n; i += kRowsMfmaThreads * 8)
      *reinterpret_cast<uint4_t*>(args.copy.dst + i) = *reinterpret_cast<const uint4_t*>(args.copy.src + i);
  }
  int pi = 0;
  int first = 0;
  for (int i = 0; i < args.n_problems - 1; ++i) {
    if (static_cast<int>(blockIdx.x) >= args.block_end[i]) {
      pi = i + 1;
      first = args.block_end[i];
    }
  }
  const LinearProblem prob = args.p[pi];
  const int blk = blockIdx.x - first;
  if (DF != RWKV_FMT_F16 && prob.fmt == DF) {  // uniform per block
    rows_mfma_block<DF, NB, G, LN, XV>(args, prob, blk, M, xs, xstride, part, &flags);
  } else {
    rows_mfma_block<RWKV_FMT_F16, NB, rows_mfma_groups_f16(G), LN, XV>(args, prob, blk, M, xs, xstride, part, &flags);
  }
}

// Formats and shapes of the few-row matrix-core launch: int8 or fp16 weights, K a multiple of 512 up to 4096 (a
// sixteenth of K in whole steps of both formats, x in LDS), N a multiple of 16.
static bool rows_mfma_shape_ok(int M, int K, int n_problems, const LinearProblem* problems) {
  if (M < 1 || M > kRowsMfmaMax || K < 1024 || K > 4096 || K % 1024 != 0) return false;
  for (int i = 0; i < n_problems; ++i) {
    const LinearProblem& p = problems[i];
    if (p.fmt != RWKV_FMT_W8 && p.fmt != RWKV_FMT_F16) return false;
    if (p.N % 16 != 0 || p.x_f32 != nullptr) return false;
  }
  return true;
}

// With the LayerNorm prologue: up to 8 rows (a staging wavefront each) of 1024 .. 4096 values, staged by half of the
// wavefronts.
static bool rows_mfma_ln_ok(int M, int K) {
  return M <= kRowsMfmaLnRows && K % 512 == 0 && M * (K / 8) <= kRowsMfmaXVecs * (kRowsMfmaThreads / 2);
}

bool linear_rows_mfma_supported(int fmt, int N, int K) {
  LinearProblem p;
  p.fmt = fmt;
  p.N = N;
  return rows_mfma_shape_ok(kRowsMfmaMin, K, 1, &p);
}

template <int DF, int NB, int G, bool LN, int XV>
static int launch_rows_mfma(hipStream_t st, LinearArgs& args, int M) {
  int total = 0;
  for (int i = 0; i < args.n_problems; ++i) {
    total += ceil_div(args.p[i].N, 16 * (args.p[i].fmt == RWKV_FMT_F16 ? rows_mfma_groups_f16(G) : G));
    args.block_end[i] = total;
  }
  const size_t lds = static_cast<size_t>(M) * (args.K + 8) * sizeof(half_t) + 16 * 256 * sizeof(float) +
                     (LN ? static_cast<size_t>(3) * args.K * sizeof(half_t) : 0);
  if (lds > 48 * 1024) {  // beyond the default limit of dynamic LDS: raised once per instantiation (to the largest M)
    static bool raised = false;
    if (!raised) {
      const size_t most = static_cast<size_t>(LN ? kRowsMfmaLnRows : kRowsMfmaMax) * (4096 + 8) * sizeof(half_t) +
                          16 * 256 * sizeof(float) + (LN ? static_cast<size_t>(3) * 4096 * sizeof(half_t) : 0);
      RWKV_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_rows_mfma_kernel<DF, NB, G, LN, XV>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(most)));
      raised = true;
    }
  }
  hipLaunchKernelGGL((linear_rows_mfma_kernel<DF, NB, G, LN, XV>), dim3(total), dim3(kRowsMfmaThreads), lds, st, args, M);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// Vectors per batch (NB) by shape: a wavefront has K * G / 1024 vectors of int8 codes to request (as many of fp16
// weights with half the groups per block, twice as many with one group) and takes them in batches of up to 16.
template <int DF, int G, bool LN, int XV>
static int launch_rows_mfma_g(hipStream_t st, LinearArgs& args, int M) {
  const int steps = args.K * G / 1024;
  if constexpr (G == 4) {
    if (steps % 16 == 0) return launch_rows_mfma<DF, 16, G, LN, XV>(st, args, M);
    if (steps % 8 == 0) return launch_rows_mfma<DF, 8, G, LN, XV>(st, args, M);
  }
  if (steps % 4 == 0) return launch_rows_mfma<DF, 4, G, LN, XV>(st, args, M);
  if (steps % 2 == 0) return launch_rows_mfma<DF, 2, G, LN, XV>(st, args, M);
  return launch_rows_mfma<DF, 1, G, LN, XV>(st, args, M);
}

template <int DF>
static int launch_rows_mfma_fmt(hipStream_t st, LinearArgs& args, int M) {
  // four groups of rows per block where that leaves no more than a quarter of the CUs without one
  int blocks4 = 0;
  for (int i = 0; i < args.n_problems; ++i)
    blocks4 += ceil_div(args.p[i].N, 16 * (args.p[i].fmt == RWKV_FMT_F16 ? rows_mfma_groups_f16(4) : 4));
  const bool g4 = blocks4 * 4 >= device_cu_count() * 3;
  constexpr int XV = kRowsMfmaXVecs;
  if (args.ln.mode != 0) {
    return g4 ? launch_rows_mfma_g<DF, 4, true, XV>(st, args, M) : launch_rows_mfma_g<DF, 1, true, XV>(st, args, M);
  }
  // the first half of the wavefronts stages x: eight vectors per thread cover 8 rows of 4096 values, sixteen all 16
  // (16 rows, 7.2B shape: 3.05 -> 2.85 ms per step against every wavefront staging its share before any request)
  if (M * (args.K / 8) <= XV * (kRowsMfmaThreads / 2)) {
    return g4 ? launch_rows_mfma_g<DF, 4, false, XV>(st, args, M) : launch_rows_mfma_g<DF, 1, false, XV>(st, args, M);
  }
  return g4 ? launch_rows_mfma_g<DF, 4, false, 2 * XV>(st, args, M) : launch_rows_mfma_g<DF, 1, false, 2 * XV>(st, args, M);
}

static int launch_rows_mfma_any(hipStream_t st, LinearArgs& args, int M, int df) {
  if (df == RWKV_FMT_W8) return launch_rows_mfma_fmt<RWKV_FMT_W8>(st, args, M);
  return launch_rows_mfma_fmt<RWKV_FMT_F16>(st, args, M);
}

int linear_rows_mfma_sliced(hipStream_t st, int fmt, int M, int N, int K, int slice, const half_t* x, const void* w,
                            float* partial, const RowCopy* copy) {
  RWKV_REQUIRE(slice > 0 && K % slice == 0 && K / slice >= 1 && K / slice <= kMaxProblems,
               "linear: %d columns in slices of %d", K, slice);
  RWKV_REQUIRE(M >= 1 && M <= kRowsMfmaMax && linear_rows_mfma_supported(fmt, N, slice),
               "linear: no few-row launch for %d rows of this format and shape (N = %d, K = %d)", M, N, slice);
  RWKV_REQUIRE(x && w && partial, "linear: NULL tensor");
  LinearArgs args = {};
  args.n_problems = K / slice;
  args.K = slice;
  args.epilogue = RWKV_EPI_NONE;
  args.out_f32 = 1;
  const int eb = fmt == RWKV_FMT_F16 ? 2 : 1;
  for (int i = 0; i < args.n_problems; ++i) {
    LinearProblem& p = args.p[i];
    p.w = static_cast<const unsigned char*>(w) + static_cast<int64_t>(i) * slice * eb;
    p.x = x + static_cast<int64_t>(i) * slice;
    p.y = partial + static_cast<int64_t>(i) * M * N;
    p.N = N;
    p.fmt = fmt;
    p.ldw = K;
    p.ldx = K;
    p.raw_f32 = 1;
  }
  if (copy && copy->n > 0) {
    RWKV_REQUIRE(copy->src && copy->dst && copy->n % 8 == 0, "linear: bad row copy");
    args.copy = *copy;
  }
  return launch_rows_mfma_any(st, args, M, fmt);
}

int linear_ln_prologue_max_rows(int K) { return K <= 4096 && K % 8 == 0 ? kRow1MaxRowsLn : 0; }

bool linear_ln_prologue_rows_ok(int fmt, int M, int N, int K) {
  if (M >= 1 && M <= linear_ln_prologue_max_rows(K)) return true;
  return M >= kRowsMfmaMin && linear_rows_mfma_supported(fmt, N, K) && rows_mfma_ln_ok(M, K);
}

// Batched small-M linear: n_problems problems sharing M (<= 8), K, epilogue and output type.
int linear_small_m(hipStream_t st, int M, int K, int n_problems, const LinearProblem* problems, int epilogue,
                   int out_f32, const LnPrologue* ln, const RowCopy* copy) {
  RWKV_REQUIRE(M >= 1 && M <= kRowsMfmaMax, "linear_small_m: M %d out of range", M);
  RWKV_REQUIRE(n_problems >= 1 && n_problems <= kMaxProblems, "linear_small_m: %d problems", n_problems);
  LinearArgs args = {};
  int max_elems = 8;
  for (int i = 0; i < n_problems; ++i) {
    const LinearProblem& p = problems[i];
    RWKV_REQUIRE(p.fmt == RWKV_FMT_F16 || p.fmt == RWKV_FMT_W8 || p.fmt == RWKV_FMT_W4,
                 "linear: unknown weight format %d", p.fmt);
    const int elems = p.fmt == RWKV_FMT_F16 ? 8 : (p.fmt == RWKV_FMT_W8 ? 16 : 32);
    max_elems = std::max(max_elems, elems);
    RWKV_REQUIRE(K > 0 && K % elems == 0, "linear: K (%d) must be a multiple of %d for this weight format", K, elems);
    if (p.fmt == RWKV_FMT_W4) RWKV_REQUIRE(K % 128 == 0, "linear: W4 needs K %% 128 == 0 (K = %d)", K);
    RWKV_REQUIRE(p.N > 0 && p.N % 4 == 0, "linear: N (%d) must be a positive multiple of 4", p.N);
    RWKV_REQUIRE(p.w && p.y && (p.x || p.x_f32 || (ln && ln->mode != 0 && p.mu)), "linear: NULL tensor");
    RWKV_REQUIRE(p.fmt == RWKV_FMT_F16 || p.scale, "linear: quantised weights need a scale tensor");
    RWKV_REQUIRE(p.fmt != RWKV_FMT_W4 || p.zp, "linear: W4 weights need a zero-point tensor");
    args.p[i] = p;
  }
  args.n_problems = n_problems;
  args.K = K;
  args.epilogue = epilogue;
  args.out_f32 = out_f32;
  // LDS tile of x: the whole K when M*K*2 bytes <= 64 KiB, else a whole number of the widest wave step
  const int step = 64 * max_elems;
  const int k_round = (K + step - 1) / step * step;
  int kt = (65536 / (2 * M)) / step * step;
  if (kt < step) kt = step;
  args.KT = std::min(kt, k_round);
  static const int rows_mfma_min = [] {
    const char* e = getenv("RWKV_ROWS_MFMA_MIN");  // tuning hook: rows from which the matrix-core launch is used
    return e ? atoi(e) : kRowsMfmaMin;
  }();
  const bool with_ln = ln && ln->mode != 0;
  const bool few_rows = M >= rows_mfma_min && rows_mfma_shape_ok(M, K, n_problems, problems) &&
                        (!with_ln || rows_mfma_ln_ok(M, K));
  if (with_ln) {
    RWKV_REQUIRE(ln->mode == 1 || ln->mode == 2, "linear: bad LayerNorm prologue mode %d", ln->mode);
    RWKV_REQUIRE(few_rows || (args.KT >= K && K % 8 == 0 &&
                              static_cast<size_t>(M) * args.KT * 2 + static_cast<size_t>(K) * 4 <= 65536),
                 "linear: LayerNorm prologue needs the whole row in LDS (M = %d, K = %d)", M, K);
    RWKV_REQUIRE(ln->x && ln->w && ln->b && ln->shift && ln->ln_out && (ln->mode == 2 ? ln->tokens != nullptr : ln->res != nullptr),
                 "linear: LayerNorm prologue has a NULL tensor");
    args.ln = *ln;
  }
  if (copy && copy->n > 0) {
    RWKV_REQUIRE(copy->src && copy->dst && copy->n % 8 == 0, "linear: bad row copy");
    args.copy = *copy;
  }
  bool gated = false;
  for (int i = 0; i < n_problems; ++i) {
    if (problems[i].x_f32 == nullptr) continue;
    gated = true;
    RWKV_REQUIRE(problems[i].x_gate != nullptr && K % 8 == 0, "linear: a gated x needs its gate and K %% 8 == 0");
  }
  if (few_rows) {
    for (int i = 0; i < n_problems; ++i)
      RWKV_REQUIRE(with_ln ? problems[i].mu != nullptr : problems[i].x != nullptr, "linear: NULL tensor");
    int df = RWKV_FMT_F16;
    for (int i = 0; i < n_problems; ++i) df = problems[i].fmt == RWKV_FMT_W8 ? RWKV_FMT_W8 : df;
    return launch_rows_mfma_any(st, args, M, df);
  }
  RWKV_REQUIRE(M <= 8, "linear: %d rows of this shape or format (K = %d) have no few-row launch", M, K);
  if (M <= (args.ln.mode != 0 ? kRow1MaxRowsLn : kRow1MaxRows)) {
    const int df = row1_format(args);
    if (df >= 0 && !(gated && args.ln.mode != 0)) {
      switch (M) {
        case 1: return launch_row1_any<1>(st, args, df);
        case 2: return launch_row1_any<2>(st, args, df);
        case 3: return launch_row1_any<3>(st, args, df);
        default: return launch_row1_any<4>(st, args, df);
      }
    }
  }
  RWKV_REQUIRE(!gated, "linear: x = x_f32 * gate is formed by launches of up to %d rows of at most 4096 values (M = %d, K = %d)",
               kRow1MaxRows, M, K);
  switch (M) {
    case 1: return launch_one<1, 2, 1>(st, args);
    case 2: return launch_one<2, 2, 1>(st, args);
    case 3: return launch_one<3, 2, 2>(st, args);
    case 4: return launch_one<4, 2, 2>(st, args);
    case 5: return launch_one<5, 4, 1>(st, args);
    case 6: return launch_one<6, 4, 1>(st, args);
    case 7: return launch_one<7, 4, 1>(st, args);
    default: return launch_one<8, 4, 1>(st, args);
  }
}

// Any M: MFMA tiles when the shape allows it and M >= 16, else row tiles of <= 8 through the GEMV kernel.
int linear_any_m(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* w, const half_t* scale,
                 const uint8_t* zp, int epilogue, int out_f32, void* y) {
  RWKV_REQUIRE(M > 0, "linear: M must be positive");
  const bool few = linear_rows_mfma_supported(fmt, N, K);
  if (M >= 16 && !(few && M <= kRowsMfmaMax) && linear_mfma_supported(fmt, M, N, K)) {
    return linear_mfma(st, fmt, M, N, K, x, w, scale, zp, epilogue, out_f32, y);
  }
  const int tile = few ? kRowsMfmaMax : 8;
  for (int m0 = 0; m0 < M; m0 += tile) {
    const int mt = std::min(tile, M - m0);
    LinearProblem p;
    p.w = w;
    p.scale = scale;
    p.zp = zp;
    p.x = x + static_cast<int64_t>(m0) * K;
    p.y = out_f32 ? static_cast<void*>(static_cast<float*>(y) + static_cast<int64_t>(m0) * N)
                  : static_cast<void*>(static_cast<half_t*>(y) + static_cast<int64_t>(m0) * N);
    p.N = N;
    p.fmt = fmt;
    const int rc = linear_small_m(st, mt, K, 1, &p, epilogue, out_f32);
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
