// Shared helpers for the gfx950 kernels: error plumbing for the C ABI, fp16 vector types,
// wave64 reductions.  Internal to the library; nothing here is exported.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdio>
#include <string>

#include "../../include/rwkv_hip.h"

namespace rwkv {

void set_error(const char* fmt, ...);
// Compute units of the current device (asked once per device; 256 if the query fails).
int device_cu_count();

inline hipStream_t as_stream(rwkv_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

#define RWKV_HIP_TRY(expr)                                                              \
  do {                                                                                  \
    hipError_t err__ = (expr);                                                          \
    if (err__ != hipSuccess) {                                                          \
      ::rwkv::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(err__), __FILE__, __LINE__); \
      return err__ == hipErrorOutOfMemory ? RWKV_E_NOMEM : RWKV_E_RUNTIME;              \
    }                                                                                   \
  } while (0)

#define RWKV_REQUIRE(cond, ...)          \
  do {                                   \
    if (!(cond)) {                       \
      ::rwkv::set_error(__VA_ARGS__);    \
      return RWKV_E_INVALID;             \
    }                                    \
  } while (0)

#define RWKV_LAUNCH_CHECK()                                                             \
  do {                                                                                  \
    hipError_t err__ = hipGetLastError();                                               \
    if (err__ != hipSuccess) {                                                          \
      ::rwkv::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(err__), __FILE__, __LINE__); \
      return RWKV_E_RUNTIME;                                                            \
    }                                                                                   \
  } while (0)

// ---- device-side types -----------------------------------------------------------------
typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kHead = 64;
constexpr float kLnEps = 1e-5f;        // include/rwkv7_fast_v4_common.hpp:24
constexpr float kLnxEps = 64.0e-5f;    // cuda/rwkv7_fast_ops_fp16.cu:17
constexpr float kKkEps = 1.0e-12f;     // cuda/rwkv7_fast_ops_fp16.cu:16

__device__ __forceinline__ float h2f(half_t h) { return static_cast<float>(h); }
__device__ __forceinline__ half_t f2h(float f) { return static_cast<half_t>(f); }  // v_cvt_f16_f32, RNE
// value after a round trip through fp16: the rounding point where the reference stores fp16
__device__ __forceinline__ float round_h(float f) { return static_cast<float>(static_cast<half_t>(f)); }

// a * b rounded to fp32 as a step of its own.  Without the barrier the compiler may fuse a product and the
// fp16 conversion that follows it into one mixed-precision instruction with a single rounding, and whether it
// does depends on the surrounding code: kernels that must agree bitwise on f16(a * b) go through this.
__device__ __forceinline__ float mul_f32(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return p;
}

// Reinterpret a dword as two fp16 values.  Always go through this by-value helper: applying
// __builtin_bit_cast directly to a vector element (`bit_cast<half2>(vec[i])`) makes this compiler read
// element 0 for every i.
__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// The reference is built with --use_fast_math (approximate division, __expf, fast tanhf); these are the
// gfx950 counterparts: v_rcp_f32 (1 ulp) and v_exp_f32.
__device__ __forceinline__ float rcp_f(float x) { return __builtin_amdgcn_rcpf(x); }
// fp32 -> fp16 as a conversion of its own.  The compiler may fold a conversion into the fma that produced the value
// (v_fma_mixlo_f16: one rounding) or keep the two apart (two roundings), by context; where two kernels, or two
// chains of one kernel, must give the same bits, both take this.
__device__ __forceinline__ half_t f2h_apart(float v) {
  asm volatile("" : "+v"(v));
  return f2h(v);
}
__device__ __forceinline__ float sigmoid_f(float x) { return rcp_f(1.0f + __expf(-x)); }
// tanh through e^(-2|x|): absolute error of a few 1e-8 (the library tanhf costs some 80 instructions)
__device__ __forceinline__ float tanh_f(float x) {
  const float t = __expf(-2.0f * fabsf(x));
  return copysignf((1.0f - t) * rcp_f(1.0f + t), x);
}

// Sum over the 64 lanes of a wave, result in every lane.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
// Sum over aligned groups of `Width` lanes (Width a power of two <= 64).
template <int Width>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = Width / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// x + (x of the lane that the DPP control CTRL pairs this lane with)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false);
  return x + __builtin_bit_cast(float, moved);
}
// Sum over the 16 lanes of a DPP row.  Every exchange is between two lanes that hold each other's operands,
// so all 16 lanes end with the bitwise same value.
__device__ __forceinline__ float row16_sum(float x) {
  x = dpp_add<0xB1>(x);   // quad_perm [1,0,3,2]
  x = dpp_add<0x4E>(x);   // quad_perm [2,3,0,1]
  x = dpp_add<0x141>(x);  // row_half_mirror: quad 0 <-> 1, 2 <-> 3
  x = dpp_add<0x140>(x);  // row_mirror: quads (0,1) <-> (3,2)
  return x;
}
// wave_sum without the trips through LDS (`__shfl_xor` is a ds_bpermute, a hundred cycles and more each, six in a
// row): the same six levels - lane i adds what lane i ^ 32, then i ^ 16, 8, 4, 2, 1 holds - so the same bits in every
// lane, with gfx950's row swaps for the two levels that cross DPP rows and DPP moves for the others.  For sums at the
// end of a wavefront's work, where nothing is left to hide that latency behind.  Every lane of the wavefront has to
// be active (a lane that is switched off would neither give nor take its value): call them from code that whole
// wavefronts run, as all their callers do.
template <bool ROWS32>
__device__ __forceinline__ float add_swapped_rows(float x) {
  // v_permlane32_swap: lanes 32-63 of the first operand change places with lanes 0-31 of the second (permlane16:
  // rows 1 and 3 of the first with rows 0 and 2 of the second); both start as x, so their sum is x[i] + x[i ^ 32]
  // (x[i ^ 16]) in every lane.  Two idle slots between a register's write and the swap that reads it.  (The
  // compiler's builtin for these returns the first operand twice.)
  float d = x, s = x;
  if constexpr (ROWS32) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(d), "+v"(s));
  } else {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(d), "+v"(s));
  }
  return d + s;
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v = add_swapped_rows<true>(v);
  v = add_swapped_rows<false>(v);
  v = dpp_add<0x128>(v);  // row_ror:8 - lane i ^ 8 of the row
  {                       // lane i ^ 4: the mirror image within eight lanes (i ^ 7), then within the quad (^ 3)
    const int m = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false);
    const int q = __builtin_amdgcn_update_dpp(0, m, 0x1B, 0xf, 0xf, false);
    v += __builtin_bit_cast(float, q);
  }
  v = dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
  v = dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]
  return v;
}

// wave_sum(a * b) as the compiler builds it where the product is formed right in front of the shuffles: the first
// level is a fused multiply-add, fma(a, b, the other lane's rounded product) - one rounding fewer than product +
// product, and so other bits.  Code that has to give the bits of such a kernel without its shuffles says it
// explicitly (wave_sum_dpp_of_product, below).

// The same butterfly for any operation on 32-bit values: lane_xor_dpp<D>(x) is what `__shfl_xor(x, D, 64)` returns.
template <int D>
__device__ __forceinline__ int lane_xor_dpp(int x) {
  static_assert(D == 32 || D == 16 || D == 8 || D == 4 || D == 2 || D == 1, "a single bit of the lane index");
  if constexpr (D == 32 || D == 16) {
    // after the swap the first operand holds x of the rows [0, 1, 0, 1] ([0, 0, 2, 2]), the second [2, 3, 2, 3] ([1, 1, 3, 3])
    int d = x, s = x;
    if constexpr (D == 32) {
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(d), "+v"(s));
    } else {
      asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(d), "+v"(s));
    }
    return (threadIdx.x & D) ? d : s;
  } else if constexpr (D == 8) {
    return __builtin_amdgcn_update_dpp(0, x, 0x128, 0xf, 0xf, false);
  } else if constexpr (D == 4) {
    return __builtin_amdgcn_update_dpp(0, __builtin_amdgcn_update_dpp(0, x, 0x141, 0xf, 0xf, false), 0x1B, 0xf, 0xf, false);
  } else if constexpr (D == 2) {
    return __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, false);
  } else {
    return __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, false);
  }
}
// v = op(v, value of lane i ^ 32), then ^ 16, 8, 4, 2, 1: every lane ends with the reduction over the wavefront
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce_dpp(T v, Op op) {
  static_assert(sizeof(T) == 4, "32-bit values");
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<32>(__builtin_bit_cast(int, v))));
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<16>(__builtin_bit_cast(int, v))));
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<8>(__builtin_bit_cast(int, v))));
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<4>(__builtin_bit_cast(int, v))));
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<2>(__builtin_bit_cast(int, v))));
  v = op(v, __builtin_bit_cast(T, lane_xor_dpp<1>(__builtin_bit_cast(int, v))));
  return v;
}

__device__ __forceinline__ float wave_sum_dpp_of_product(float a, float b) {
  float p;
  {
#pragma clang fp contract(off)
    p = a * b;
  }
  float v = fmaf(a, b, __builtin_bit_cast(float, lane_xor_dpp<32>(__builtin_bit_cast(int, p))));
  v = add_swapped_rows<false>(v);
  v = dpp_add<0x128>(v);
  v += __builtin_bit_cast(float, lane_xor_dpp<4>(__builtin_bit_cast(int, v)));
  v = dpp_add<0x4E>(v);
  v = dpp_add<0xB1>(v);
  return v;
}

// Sum over the 64 lanes of a wave without index registers (DPP inside the four rows, then the four row sums through
// scalar registers); the result is wave-uniform.  For kernels that are short of vector registers.
__device__ __forceinline__ float wave_sum_uniform(float v) {
  const int r = __builtin_bit_cast(int, row16_sum(v));
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(r, 48));
  return (a + b) + (c + d);
}
// `scratch` (NW floats of LDS) must not be in use by an earlier call that some wave may still be reading: give
// consecutive calls their own scratch.
template <int NW>
__device__ __forceinline__ float block_sum_uniform(float v, float* scratch) {
  v = wave_sum_uniform(v);
  if constexpr (NW == 1) return v;
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += scratch[i];
  return t;
}

// Block-wide sum for blocks of NW waves; `scratch` holds NW floats of LDS.  All threads get the sum.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum_dpp(v);
  if constexpr (NW == 1) return v;
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // scratch may still be read from a previous call
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += scratch[i];
  return t;
}

inline int ceil_div(int64_t a, int64_t b) { return static_cast<int>((a + b - 1) / b); }

}  // namespace rwkv
