// TEST INFRASTRUCTURE ONLY -- scalar CPU restatement of the RWKV-7 inference hot path.
// See rwkv_oracle.h for the contract and for what pins each function.  Plain C++17, no SIMD
// intrinsics; fp32 arithmetic with explicit fp16 rounding points where the reference's
// kernels write fp16 to memory.  Reference citations are relative to the reference repo root.
#include "rwkv_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <thread>
#include <vector>

namespace {

int g_threads = 1;

// Runs fn(i) for i in [0,n) on g_threads std::threads (contiguous ranges).  Units must be independent.
void parallel_for(int64_t n, const std::function<void(int64_t)>& fn) {
  const int nt = static_cast<int>(std::min<int64_t>(g_threads, n));
  if (nt <= 1) {
    for (int64_t i = 0; i < n; ++i) fn(i);
    return;
  }
  std::vector<std::thread> pool;
  pool.reserve(nt);
  for (int t = 0; t < nt; ++t) {
    const int64_t lo = n * t / nt;
    const int64_t hi = n * (t + 1) / nt;
    pool.emplace_back([lo, hi, &fn]() {
      for (int64_t i = lo; i < hi; ++i) fn(i);
    });
  }
  for (auto& th : pool) th.join();
}

// fp16 -> fp32 through a 65536-entry table (filled from orc_f16_to_f32 on first use)
struct HalfTable {
  float v[65536];
  HalfTable() {
    for (uint32_t i = 0; i < 65536; ++i) v[i] = orc_f16_to_f32(static_cast<uint16_t>(i));
  }
};
inline float h2f(uint16_t h) {
  static const HalfTable table;
  return table.v[h];
}
inline uint16_t f2h(float x) { return orc_f32_to_f16(x); }

inline float sigmoidf_(float x) { return 1.0f / (1.0f + std::exp(-x)); }

constexpr int kHead = 64;

}  // namespace

// All orc_* functions get C linkage from their declarations in rwkv_oracle.h.

void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_threads(void) { return g_threads; }

// ---------------------------------------------------------------------------------------------
// fp16 conversion.  The reference's kernels round with __float2half_rn (round-to-nearest-even),
// e.g. cuda/rwkv7_fast_ops_fp16.cu:33-39; its host-side table (src/pth_tensor.cpp:651-720) is
// only used at load time.  This is IEEE binary16 RNE with subnormals, pinned against numpy.
// ---------------------------------------------------------------------------------------------
float orc_f16_to_f32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t mant = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (mant == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        ++e;
        mant <<= 1;
      } while ((mant & 0x400u) == 0);
      bits = sign | (static_cast<uint32_t>(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (mant << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (mant << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

uint16_t orc_f32_to_f16(float x) {
  uint32_t bits;
  std::memcpy(&bits, &x, 4);
  const uint16_t sign = static_cast<uint16_t>((bits >> 16) & 0x8000u);
  const uint32_t absb = bits & 0x7fffffffu;
  if (absb >= 0x7f800000u) {  // inf / nan
    return static_cast<uint16_t>(sign | (absb > 0x7f800000u ? 0x7e00u : 0x7c00u));
  }
  if (absb >= 0x477ff000u) {  // >= 65520 rounds to inf
    return static_cast<uint16_t>(sign | 0x7c00u);
  }
  if (absb < 0x38800000u) {  // below 2^-14: subnormal half or zero
    if (absb < 0x33000000u) {  // below 2^-25: rounds to zero (2^-25 itself ties to even = 0)
      return sign;
    }
    const int exp = static_cast<int>(absb >> 23);            // biased fp32 exponent
    const uint32_t mant = (absb & 0x7fffffu) | 0x800000u;    // 24-bit significand
    const int shift = 126 - exp;                             // value = mant * 2^(exp-150); half sub unit 2^-24
    // result = round(mant * 2^(exp-150+24)) = round(mant >> shift), shift in [14,24]
    const uint32_t q = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    uint32_t r = q;
    if (rem > half || (rem == half && (q & 1u))) ++r;
    return static_cast<uint16_t>(sign | r);
  }
  // normal range
  const uint32_t exp = (absb >> 23) - 112u;  // half biased exponent, 1..30
  const uint32_t mant = absb & 0x7fffffu;
  uint32_t r = (exp << 10) | (mant >> 13);
  const uint32_t rem = mant & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;  // carry may bump the exponent; that is correct
  return static_cast<uint16_t>(sign | r);
}

void orc_f32_to_f16_array(const float* src, uint16_t* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = orc_f32_to_f16(src[i]);
}
void orc_f16_to_f32_array(const uint16_t* src, float* dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = orc_f16_to_f32(src[i]);
}

// ---------------------------------------------------------------------------------------------
// Checkpoint tensors, bf16 -> fp16.  cuda/rwkv7_v3a_ops.cu:70-116 (bf16_bits_to_float_dev, bf16_to_f16_kernel,
// bf16_to_f16_transpose_kernel): the bf16 pattern is the upper half of an fp32, the fp16 is that fp32 rounded to
// nearest even.  :153-185 (emb_ln0_bf16_to_f16_kernel): per embedding row, mean and variance in fp32 over the
// widened values (two passes), y = f16((x - mean) * rstd * w + b) with w, b widened from bf16.  Sums run
// c = 0..C-1 in order (the kernel's own order over 256 threads is not restated: tolerance-level only).
// ---------------------------------------------------------------------------------------------
static inline float bf16_widen(uint16_t bits) {
  const uint32_t wide = static_cast<uint32_t>(bits) << 16;
  float f;
  std::memcpy(&f, &wide, sizeof(f));
  return f;
}

void orc_bf16_to_f16(int rows, int cols, int transpose, const uint16_t* src, uint16_t* dst) {
  for (int r = 0; r < rows; ++r) {
    for (int c = 0; c < cols; ++c) {
      const uint16_t h = orc_f32_to_f16(bf16_widen(src[static_cast<int64_t>(r) * cols + c]));
      if (transpose) {
        dst[static_cast<int64_t>(c) * rows + r] = h;
      } else {
        dst[static_cast<int64_t>(r) * cols + c] = h;
      }
    }
  }
}

void orc_emb_ln0(int V, int C, const uint16_t* emb, const uint16_t* w, const uint16_t* b, float eps, uint16_t* out) {
  parallel_for(V, [&](int64_t v) {
    const uint16_t* row = emb + v * C;
    float sum = 0.0f;
    for (int c = 0; c < C; ++c) sum += bf16_widen(row[c]);
    const float mean = sum / static_cast<float>(C);
    float sq = 0.0f;
    for (int c = 0; c < C; ++c) {
      const float d = bf16_widen(row[c]) - mean;
      sq += d * d;
    }
    const float rstd = 1.0f / std::sqrt(sq / static_cast<float>(C) + eps);
    for (int c = 0; c < C; ++c) {
      out[v * C + c] = orc_f32_to_f16((bf16_widen(row[c]) - mean) * rstd * bf16_widen(w[c]) + bf16_widen(b[c]));
    }
  });
}

// ---------------------------------------------------------------------------------------------
// WKV7.  cuda/rwkv7_wkv_fp32_v2.cu:13-14,26-28 (decay map), :100-126 (per-token recurrence of
// wkv_fp32_v2_kernel): thread i owns state row i;
//   sa = sum_j S[i][j]*a[j];  S[i][j] = S[i][j]*d[j] + sa*b[j] + k[j]*v[i];  y[i] = sum_j S[i][j]*r[j].
// State layout [B,H,64,64] as in :86.  Sums run j = 0..63 in order, in fp32.
// ---------------------------------------------------------------------------------------------
static inline float wkv_decay(float w, int w_mode) {
  if (w_mode == 1) return w;
  // exp2f(W_SCALE_LOG2_E / (1 + exp2f(NLOG2_E * w)))  ==  exp(-e^{-1/2} * sigmoid(w))
  return std::exp2(-0.8750387749145276f / (1.0f + std::exp2(-1.4426950408889634f * w)));
}

template <typename LoadF, typename StoreF>
static void wkv7_impl(int B, int T, int C, int H, int w_mode, float* state, LoadF ld, StoreF st) {
  parallel_for(static_cast<int64_t>(B) * H, [&](int64_t bh) {
    const int b = static_cast<int>(bh / H);
    const int h = static_cast<int>(bh % H);
    float* S = state + bh * kHead * kHead;
    float r[kHead], d[kHead], k[kHead], a[kHead], bb[kHead];
    for (int t = 0; t < T; ++t) {
      const int64_t base = (static_cast<int64_t>(b) * T + t) * C + h * kHead;
      for (int j = 0; j < kHead; ++j) {
        r[j] = ld(0, base + j);
        d[j] = wkv_decay(ld(1, base + j), w_mode);
        k[j] = ld(2, base + j);
        a[j] = ld(4, base + j);
        bb[j] = ld(5, base + j);
      }
      for (int i = 0; i < kHead; ++i) {
        float* row = S + i * kHead;
        float sa = 0.0f;
        for (int j = 0; j < kHead; ++j) sa += row[j] * a[j];
        const float vi = ld(3, base + i);
        float y = 0.0f;
        for (int j = 0; j < kHead; ++j) {
          float s = row[j];
          s = s * d[j] + sa * bb[j] + k[j] * vi;
          y += s * r[j];
          row[j] = s;
        }
        st(base + i, y);
      }
    }
  });
}

void orc_wkv7_f32(int B, int T, int C, int H, int w_mode, float* state, const float* r, const float* w,
                  const float* k, const float* v, const float* a, const float* b, float* y) {
  const float* in[6] = {r, w, k, v, a, b};
  wkv7_impl(B, T, C, H, w_mode, state, [&](int which, int64_t idx) { return in[which][idx]; },
            [&](int64_t idx, float val) { y[idx] = val; });
}

void orc_wkv7_f16(int B, int T, int C, int H, int w_mode, float* state, const uint16_t* r, const uint16_t* w,
                  const uint16_t* k, const uint16_t* v, const uint16_t* a, const uint16_t* b, uint16_t* y) {
  const uint16_t* in[6] = {r, w, k, v, a, b};
  wkv7_impl(B, T, C, H, w_mode, state, [&](int which, int64_t idx) { return h2f(in[which][idx]); },
            [&](int64_t idx, float val) { y[idx] = f2h(val); });
}

// ---------------------------------------------------------------------------------------------
// WKV7 with the state kept in fp16 (the reference server's default mode).  cuda/rwkv7_wkv_fp16_v2.cu; the per-token
// arithmetic is the same in every kernel of that file (:157-193, :342-367, :433-468, :531-556, :632-660).  Thread i
// owns state row i as 32 half2 pairs; every operation is an fp16 fused multiply-add with one rounding (__hfma2):
//   sa2    = chain over pairs j = 0..31 of  fma(a[j], S[i][j], sa2)      (even columns in .x, odd columns in .y)
//   sa     = f16(sa2.x + sa2.y)
//   wd[c]  = f16(exp2f(NEXP_HALF_LOG2_E / (1 + exp2f(NLOG2_E * w))) - 1 + rotator1(elapsed[b] + h*64 + c + t))  (:41-52)
//            with w = float(w_raw[c]) (+ float(w0[c]) when w0 is given: the sum is not rounded to fp16)
//   S[i][c] = fma(S[i][c], wd[c], fma(k[c], v[i], fma(sa, b[c], S[i][c])))   i.e. S*(d-1) + (k*v + (sa*b + S))
//   y2     = chain over pairs of  fma(S'[i][j], r[j], y2);   y[i] = f16(y2.x + y2.y)
// rotator1(x) = 2^-41 * float(int32(ROT1 * x)), ROT1 = int32(2654435769): a dither below fp16 resolution of d - 1
// that makes the rounding of the decay unbiased over consecutive tokens and channels.
// fp16 fma: the exact product of two halves and the sum with a third fit a double (or differ from it by less than
// what could move a rounding boundary), so rounding the double result to fp16 once is the fused operation.
// ---------------------------------------------------------------------------------------------
uint16_t orc_f64_to_f16(double x) {
  uint64_t bits;
  std::memcpy(&bits, &x, sizeof(bits));
  const uint16_t sign = static_cast<uint16_t>((bits >> 48) & 0x8000u);
  if (std::isnan(x)) return static_cast<uint16_t>(sign | 0x7e00u);
  const double ax = std::fabs(x);
  if (ax >= 65520.0) return static_cast<uint16_t>(sign | 0x7c00u);  // 65504 + half an ulp ties to even = infinity
  if (ax < 6.103515625e-05) {                                       // below 2^-14: multiples of 2^-24
    const double q = std::nearbyint(ax * 16777216.0);               // round to nearest even (default mode)
    return static_cast<uint16_t>(sign | static_cast<uint16_t>(q));  // q == 1024 is the smallest normal number
  }
  int e;
  (void)std::frexp(ax, &e);  // ax = m * 2^e, m in [0.5, 1)
  e -= 1;                    // ax in [2^e, 2^(e+1))
  double mant = std::nearbyint(std::ldexp(ax, 10 - e));  // in [1024, 2048]
  if (mant >= 2048.0) {
    mant = 1024.0;
    e += 1;
  }
  return static_cast<uint16_t>(sign | static_cast<uint16_t>((e + 15) << 10) | (static_cast<uint16_t>(mant) - 1024u));
}

static inline uint16_t hfma16(uint16_t a, uint16_t b, uint16_t c) {
  return orc_f64_to_f16(static_cast<double>(h2f(a)) * static_cast<double>(h2f(b)) + static_cast<double>(h2f(c)));
}
static inline uint16_t hadd16(uint16_t a, uint16_t b) {
  return orc_f64_to_f16(static_cast<double>(h2f(a)) + static_cast<double>(h2f(b)));
}

uint16_t orc_f16_fma(uint16_t a, uint16_t b, uint16_t c) { return hfma16(a, b, c); }

float orc_wkv16_rotator(int32_t x) {
  const uint32_t prod = 2654435769u * static_cast<uint32_t>(x);  // int32 multiplication that wraps
  int32_t sp;
  std::memcpy(&sp, &prod, sizeof(sp));
  return 4.547473508864641e-13f * static_cast<float>(sp);
}

uint16_t orc_wkv16_w_delta(uint16_t w_raw, const uint16_t* w0, int c, int32_t phase) {
  float w = h2f(w_raw);
  if (w0) w += h2f(w0[c]);
  const float d = std::exp2(-0.8750387749145276f / (1.0f + std::exp2(-1.4426950408889634f * w))) - 1.0f + orc_wkv16_rotator(phase);
  return f2h(d);
}

void orc_wkv7_f16state(int B, int T, int C, int H, uint16_t* state, const uint16_t* r, const uint16_t* w,
                       const uint16_t* w0, const uint16_t* k, const uint16_t* v, const uint16_t* a,
                       const uint16_t* b, uint16_t* y, const int32_t* elapsed) {
  parallel_for(static_cast<int64_t>(B) * H, [&](int64_t bh) {
    const int bi = static_cast<int>(bh / H);
    const int h = static_cast<int>(bh % H);
    uint16_t* S = state + bh * kHead * kHead;
    uint16_t wd[kHead];
    for (int t = 0; t < T; ++t) {
      const int64_t base = (static_cast<int64_t>(bi) * T + t) * C + h * kHead;
      for (int c = 0; c < kHead; ++c) wd[c] = orc_wkv16_w_delta(w[base + c], w0, h * kHead + c, elapsed[bi] + h * kHead + c + t);
      for (int i = 0; i < kHead; ++i) {
        uint16_t* row = S + i * kHead;
        uint16_t sa_even = 0, sa_odd = 0;
        for (int j = 0; j < kHead / 2; ++j) {
          sa_even = hfma16(a[base + 2 * j], row[2 * j], sa_even);
          sa_odd = hfma16(a[base + 2 * j + 1], row[2 * j + 1], sa_odd);
        }
        const uint16_t sa = hadd16(sa_even, sa_odd);
        const uint16_t vi = v[base + i];
        uint16_t y_even = 0, y_odd = 0;
        for (int j = 0; j < kHead / 2; ++j) {
          for (int q = 0; q < 2; ++q) {
            const int c = 2 * j + q;
            const uint16_t s = row[c];
            const uint16_t s_new = hfma16(s, wd[c], hfma16(k[base + c], vi, hfma16(sa, b[base + c], s)));
            row[c] = s_new;
            if (q == 0) y_even = hfma16(s_new, r[base + c], y_even);
            else y_odd = hfma16(s_new, r[base + c], y_odd);
          }
        }
        y[base + i] = hadd16(y_even, y_odd);
      }
    }
  });
}

// ---------------------------------------------------------------------------------------------
// Weight formats.  The reference has no quantised path (fp16 weights only, e.g.
// cuda/rwkv7_v3a_ops.cu:464-560); these formats are this project's own and are unpinned at
// the reference boundary.  Fixed operation order so a device implementation can be bit-exact:
//   W8: amax = max|w| (fp32);  s = f16(amax / 127);  q = clamp(rint(w / f32(s)), -127, 127); s==0 -> q=0
//       dequant = f16(f32(s) * q)
//   W4: per 128-wide group along K:  lo = min(min w, 0), hi = max(max w, 0);  s = f16((hi-lo)/15);
//       s==0 -> s=1;  zp = clamp(rint(-lo / f32(s)), 0, 15);  q = clamp(rint(w / f32(s)) + zp, 0, 15)
//       dequant = f16(f32(s) * (q - zp))
// ---------------------------------------------------------------------------------------------
void orc_quantize_w8(int N, int K, const uint16_t* w, int8_t* q, uint16_t* scale) {
  parallel_for(N, [&](int64_t n) {
    const uint16_t* row = w + n * K;
    float amax = 0.0f;
    for (int k = 0; k < K; ++k) amax = std::max(amax, std::fabs(h2f(row[k])));
    const uint16_t sh = f2h(amax / 127.0f);
    scale[n] = sh;
    const float s = h2f(sh);
    for (int k = 0; k < K; ++k) {
      float v = 0.0f;
      if (s > 0.0f) v = std::nearbyint(h2f(row[k]) / s);
      v = std::min(127.0f, std::max(-127.0f, v));
      q[n * K + k] = static_cast<int8_t>(v);
    }
  });
}

void orc_dequant_w8(int N, int K, const int8_t* q, const uint16_t* scale, uint16_t* w) {
  parallel_for(N, [&](int64_t n) {
    const float s = h2f(scale[n]);
    for (int k = 0; k < K; ++k) w[n * K + k] = f2h(s * static_cast<float>(q[n * K + k]));
  });
}

void orc_quantize_w4(int N, int K, const uint16_t* w, uint8_t* q, uint16_t* scale, uint8_t* zp) {
  const int G = K / 128;
  parallel_for(N, [&](int64_t n) {
    for (int g = 0; g < G; ++g) {
      const uint16_t* grp = w + n * K + g * 128;
      float lo = 0.0f, hi = 0.0f;
      for (int k = 0; k < 128; ++k) {
        const float v = h2f(grp[k]);
        lo = std::min(lo, v);
        hi = std::max(hi, v);
      }
      uint16_t sh = f2h((hi - lo) / 15.0f);
      if (h2f(sh) == 0.0f) sh = f2h(1.0f);
      const float s = h2f(sh);
      float z = std::nearbyint(-lo / s);
      z = std::min(15.0f, std::max(0.0f, z));
      scale[n * G + g] = sh;
      zp[n * G + g] = static_cast<uint8_t>(z);
      for (int k = 0; k < 128; k += 2) {
        uint8_t code[2];
        for (int e = 0; e < 2; ++e) {
          float c = std::nearbyint(h2f(grp[k + e]) / s) + z;
          c = std::min(15.0f, std::max(0.0f, c));
          code[e] = static_cast<uint8_t>(c);
        }
        q[(n * K + g * 128 + k) / 2] = static_cast<uint8_t>(code[0] | (code[1] << 4));
      }
    }
  });
}

void orc_dequant_w4(int N, int K, const uint8_t* q, const uint16_t* scale, const uint8_t* zp, uint16_t* w) {
  const int G = K / 128;
  parallel_for(N, [&](int64_t n) {
    for (int k = 0; k < K; ++k) {
      const int g = k / 128;
      const uint8_t byte = q[(n * K + k) / 2];
      const int code = (k & 1) ? (byte >> 4) : (byte & 15);
      const float s = h2f(scale[n * G + g]);
      w[n * K + k] = f2h(s * static_cast<float>(code - static_cast<int>(zp[n * G + g])));
    }
  });
}

// ---------------------------------------------------------------------------------------------
// GEMV / small-M GEMM, y = x . W^T with W [N,K] ("orig" layout), fp32 accumulate, f16 result:
// cuda/rwkv7_v3a_ops.cu:464-560 (linear_orig_row1_exact_f16_kernel).  For the quantised formats
// the integer codes are accumulated against x in fp32 and the scale is applied once per row
// (W8) or once per 128-group (W4) -- mathematically sum_k dequant(q)*x without rounding each
// dequantised weight to fp16.
// ---------------------------------------------------------------------------------------------
static float dot_row(int fmt, int K, const uint16_t* x, const void* w, int64_t n, const uint16_t* scale,
                     const uint8_t* zp) {
  if (fmt == ORC_FMT_F16) {
    const uint16_t* row = static_cast<const uint16_t*>(w) + n * K;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc += h2f(x[k]) * h2f(row[k]);
    return acc;
  }
  if (fmt == ORC_FMT_W8) {
    const int8_t* row = static_cast<const int8_t*>(w) + n * K;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc += h2f(x[k]) * static_cast<float>(row[k]);
    return acc * h2f(scale[n]);
  }
  const int G = K / 128;
  const uint8_t* row = static_cast<const uint8_t*>(w) + n * (K / 2);
  float acc = 0.0f;
  for (int g = 0; g < G; ++g) {
    const float z = static_cast<float>(zp[n * G + g]);
    float part = 0.0f;
    for (int k = 0; k < 128; ++k) {
      const int kk = g * 128 + k;
      const uint8_t byte = row[kk / 2];
      const int code = (kk & 1) ? (byte >> 4) : (byte & 15);
      part += h2f(x[kk]) * (static_cast<float>(code) - z);
    }
    acc += part * h2f(scale[n * G + g]);
  }
  return acc;
}

void orc_gemv_any_f32(int fmt, int M, int N, int K, const uint16_t* x, const void* w, const uint16_t* scale,
                      const uint8_t* zp, float* y) {
  parallel_for(N, [&](int64_t n) {
    for (int m = 0; m < M; ++m) y[static_cast<int64_t>(m) * N + n] = dot_row(fmt, K, x + static_cast<int64_t>(m) * K, w, n, scale, zp);
  });
}

static void gemv_any_f16(int fmt, int M, int N, int K, const uint16_t* x, const void* w, const uint16_t* scale,
                         const uint8_t* zp, uint16_t* y) {
  parallel_for(N, [&](int64_t n) {
    for (int m = 0; m < M; ++m)
      y[static_cast<int64_t>(m) * N + n] = f2h(dot_row(fmt, K, x + static_cast<int64_t>(m) * K, w, n, scale, zp));
  });
}

void orc_gemv_f16(int M, int N, int K, const uint16_t* x, const uint16_t* w, uint16_t* y) {
  gemv_any_f16(ORC_FMT_F16, M, N, K, x, w, nullptr, nullptr, y);
}
void orc_gemv_w8(int M, int N, int K, const uint16_t* x, const int8_t* q, const uint16_t* scale, uint16_t* y) {
  gemv_any_f16(ORC_FMT_W8, M, N, K, x, q, scale, nullptr, y);
}
void orc_gemv_w4(int M, int N, int K, const uint16_t* x, const uint8_t* q, const uint16_t* scale,
                 const uint8_t* zp, uint16_t* y) {
  gemv_any_f16(ORC_FMT_W4, M, N, K, x, q, scale, zp, y);
}

// ---------------------------------------------------------------------------------------------
// LayerNorm family.  Two-pass mean/variance in fp32, rstd = 1/sqrt(var+eps):
// cuda/rwkv7_v3a_ops.cu:1272-1308 (layer_norm), :1310-1351 (add+LN; the LN reads the unrounded
// fp32 sum while x_out is the rounded sum), :1800-1931 (add + last-token LN),
// :1933-1985 (add+LN+cmix lerp; the lerp reads the fp16-ROUNDED LN output, :1978-1983),
// :1987-2060 (add+LN+6 lerps).
// ---------------------------------------------------------------------------------------------
static void ln_row(int C, const float* v, const uint16_t* w, const uint16_t* b, float eps, uint16_t* y) {
  float sum = 0.0f;
  for (int c = 0; c < C; ++c) sum += v[c];
  const float mean = sum / static_cast<float>(C);
  float sv = 0.0f;
  for (int c = 0; c < C; ++c) {
    const float d = v[c] - mean;
    sv += d * d;
  }
  const float rstd = 1.0f / std::sqrt(sv / static_cast<float>(C) + eps);
  for (int c = 0; c < C; ++c) y[c] = f2h((v[c] - mean) * rstd * h2f(w[c]) + h2f(b[c]));
}

void orc_layer_norm(int rows, int C, const uint16_t* x, const uint16_t* w, const uint16_t* b, uint16_t* y,
                    float eps) {
  parallel_for(rows, [&](int64_t r) {
    std::vector<float> v(C);
    for (int c = 0; c < C; ++c) v[c] = h2f(x[r * C + c]);
    ln_row(C, v.data(), w, b, eps, y + r * C);
  });
}

void orc_add_layer_norm(int rows, int C, const uint16_t* x, const uint16_t* res, const uint16_t* w,
                        const uint16_t* b, uint16_t* x_out, uint16_t* y, float eps) {
  parallel_for(rows, [&](int64_t r) {
    std::vector<float> v(C);
    for (int c = 0; c < C; ++c) v[c] = h2f(x[r * C + c]) + h2f(res[r * C + c]);
    ln_row(C, v.data(), w, b, eps, y + r * C);
    for (int c = 0; c < C; ++c) x_out[r * C + c] = f2h(v[c]);
  });
}

void orc_add_last_layer_norm(int B, int T, int C, const uint16_t* x, const uint16_t* res, const uint16_t* w,
                             const uint16_t* b, uint16_t* y, float eps) {
  for (int bi = 0; bi < B; ++bi) {
    const int64_t src = (static_cast<int64_t>(bi) * T + (T - 1)) * C;
    std::vector<float> v(C);
    for (int c = 0; c < C; ++c) v[c] = h2f(x[src + c]) + h2f(res[src + c]);
    ln_row(C, v.data(), w, b, eps, y + static_cast<int64_t>(bi) * C);
  }
}

// Token shift: cuda/rwkv7_fast_ops_fp16.cu:53-109 (tmix_mix6), :393-419 (cmix_mix),
// :111-127 (shift <- x[T-1]).  out = cur + (prev - cur) * mu in fp32, rounded to fp16.
void orc_token_shift_mix(int B, int T, int C, int n_mix, const uint16_t* x, uint16_t* shift,
                         const uint16_t* const* mu, uint16_t* const* out) {
  for (int b = 0; b < B; ++b) {
    for (int t = 0; t < T; ++t) {
      const int64_t idx = (static_cast<int64_t>(b) * T + t) * C;
      for (int c = 0; c < C; ++c) {
        const float cur = h2f(x[idx + c]);
        const float prev = (t == 0) ? h2f(shift[static_cast<int64_t>(b) * C + c]) : h2f(x[idx - C + c]);
        const float dx = prev - cur;
        for (int s = 0; s < n_mix; ++s) out[s][idx + c] = f2h(cur + dx * h2f(mu[s][c]));
      }
    }
  }
  for (int b = 0; b < B; ++b)
    for (int c = 0; c < C; ++c)
      shift[static_cast<int64_t>(b) * C + c] = x[(static_cast<int64_t>(b) * T + (T - 1)) * C + c];
}

void orc_add_layer_norm_cmix_mix(int rows, int C, const uint16_t* x, const uint16_t* res, uint16_t* shift,
                                 const uint16_t* w, const uint16_t* b, const uint16_t* mu_k, uint16_t* x_out,
                                 uint16_t* mixed, float eps) {
  std::vector<uint16_t> y(static_cast<size_t>(rows) * C);
  orc_add_layer_norm(rows, C, x, res, w, b, x_out, y.data(), eps);
  for (int64_t i = 0; i < static_cast<int64_t>(rows) * C; ++i) {
    const float yv = h2f(y[i]);
    const float prev = h2f(shift[i]);
    mixed[i] = f2h(yv + (prev - yv) * h2f(mu_k[i % C]));
    shift[i] = y[i];
  }
}

void orc_add_layer_norm_tmix_mix6(int rows, int C, const uint16_t* x, const uint16_t* res, uint16_t* shift,
                                  const uint16_t* w, const uint16_t* b, const uint16_t* const* mu6,
                                  uint16_t* x_out, uint16_t* const* out6, float eps) {
  std::vector<uint16_t> y(static_cast<size_t>(rows) * C);
  orc_add_layer_norm(rows, C, x, res, w, b, x_out, y.data(), eps);
  for (int64_t i = 0; i < static_cast<int64_t>(rows) * C; ++i) {
    const float yv = h2f(y[i]);
    const float dx = h2f(shift[i]) - yv;
    for (int s = 0; s < 6; ++s) out6[s][i] = f2h(yv + dx * h2f(mu6[s][i % C]));
    shift[i] = y[i];
  }
}

// cuda/rwkv7_fast_ops_fp16.cu:129-172 (tmix_kk_a_gate_kernel):
//   u = k*k_k; kk = u / max(||u||_2, 1e-12) per 64-channel head; a = sigmoid(a0 + a12);
//   new_k = k * (a*k_a + (1 - k_a)); neg_kk = -kk; kka = kk*a.
void orc_kk_a_gate(int rows, int C, int H, const uint16_t* k, const uint16_t* k_k, const uint16_t* a0,
                   const uint16_t* a12, const uint16_t* k_a, uint16_t* new_k, uint16_t* neg_kk, uint16_t* kka) {
  (void)C;
  for (int64_t rh = 0; rh < static_cast<int64_t>(rows) * H; ++rh) {
    const int h = static_cast<int>(rh % H);
    const int64_t base = rh * kHead;
    float u[kHead];
    float ss = 0.0f;
    for (int j = 0; j < kHead; ++j) {
      u[j] = h2f(k[base + j]) * h2f(k_k[h * kHead + j]);
      ss += u[j] * u[j];
    }
    const float inv = 1.0f / std::max(std::sqrt(ss), 1.0e-12f);
    for (int j = 0; j < kHead; ++j) {
      const int c = h * kHead + j;
      const float kk = u[j] * inv;
      const float av = sigmoidf_(h2f(a0[c]) + h2f(a12[base + j]));
      const float ka = h2f(k_a[c]);
      new_k[base + j] = f2h(h2f(k[base + j]) * (av * ka + (1.0f - ka)));
      neg_kk[base + j] = f2h(-kk);
      kka[base + j] = f2h(kk * av);
    }
  }
}

// cuda/rwkv7_fast_ops_fp16.cu:174-237 (tmix_lnx_rkvres_xg_kernel): per-head GroupNorm with
// eps 64e-5 (:17), + (sum_head r*k*r_k) * v, times g.
void orc_lnx_rkvres_xg(int rows, int C, int H, const uint16_t* y, const uint16_t* r, const uint16_t* k,
                       const uint16_t* v, const uint16_t* r_k, const uint16_t* lnw, const uint16_t* lnb,
                       const uint16_t* g, uint16_t* out) {
  (void)C;
  for (int64_t rh = 0; rh < static_cast<int64_t>(rows) * H; ++rh) {
    const int h = static_cast<int>(rh % H);
    const int64_t base = rh * kHead;
    float sum = 0.0f;
    for (int j = 0; j < kHead; ++j) sum += h2f(y[base + j]);
    const float mean = sum * (1.0f / 64.0f);
    float ss = 0.0f, dot = 0.0f;
    for (int j = 0; j < kHead; ++j) {
      const float d = h2f(y[base + j]) - mean;
      ss += d * d;
      dot += h2f(r[base + j]) * h2f(k[base + j]) * h2f(r_k[h * kHead + j]);
    }
    const float rstd = 1.0f / std::sqrt(ss * (1.0f / 64.0f) + 64.0e-5f);
    for (int j = 0; j < kHead; ++j) {
      const int c = h * kHead + j;
      const float d = h2f(y[base + j]) - mean;
      const float o = (d * rstd * h2f(lnw[c]) + h2f(lnb[c]) + dot * h2f(v[base + j])) * h2f(g[base + j]);
      out[base + j] = f2h(o);
    }
  }
}

// cuda/rwkv7_v3a_ops.cu:1118-1123 (fused LoRA-out epilogue): the gate reads the unrounded
// fp32 LoRA sum; out = v + (v_first - v) * sigmoid(v0 + v12).
void orc_vres_gate(int rows, int C, const uint16_t* v, const uint16_t* v_first, const uint16_t* v0,
                   const float* v12, uint16_t* out) {
  for (int64_t i = 0; i < static_cast<int64_t>(rows) * C; ++i) {
    const float vv = h2f(v[i]);
    const float gate = sigmoidf_(h2f(v0[i % C]) + v12[i]);
    out[i] = f2h(vv + (h2f(v_first[i]) - vv) * gate);
  }
}

// cuda/rwkv7_fast_ops_fp16.cu:421-434 and :636-639: relu then square in fp32, rounded to fp16.
void orc_relu_square(int64_t n, const uint16_t* x, uint16_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    const float v = std::max(h2f(x[i]), 0.0f);
    out[i] = f2h(v * v);
  }
}

// cuda/rwkv7_fast_ops_fp16.cu:462-477 (w_raw = w12 + w0).
void orc_add_vec(int rows, int C, const uint16_t* x, const uint16_t* vec, uint16_t* out) {
  for (int64_t i = 0; i < static_cast<int64_t>(rows) * C; ++i) out[i] = f2h(h2f(x[i]) + h2f(vec[i % C]));
}

// LoRA pair: cuda/rwkv7_v3a_ops.cu:873-940 (rank-in: fp32 dot, fp16 result) and :1027-1130
// (rank-out: activation applied to the fp16 hidden in fp32, unrounded; fp32 dot).
void orc_lora(int rows, int C, int R, int act, const uint16_t* x, const uint16_t* w1, const uint16_t* w2,
              float* out_f32) {
  for (int m = 0; m < rows; ++m) {
    std::vector<float> hid(R);
    for (int r = 0; r < R; ++r) {
      float acc = 0.0f;
      for (int c = 0; c < C; ++c) acc += h2f(x[static_cast<int64_t>(m) * C + c]) * h2f(w1[static_cast<int64_t>(r) * C + c]);
      float hv = h2f(f2h(acc));
      if (act == 1) hv = std::tanh(hv);
      if (act == 2) hv = sigmoidf_(hv);
      hid[r] = hv;
    }
    parallel_for(C, [&](int64_t c) {
      float acc = 0.0f;
      for (int r = 0; r < R; ++r) acc += hid[r] * h2f(w2[c * R + r]);
      out_f32[static_cast<int64_t>(m) * C + c] = acc;
    });
  }
}

// ---------------------------------------------------------------------------------------------
// Sampler, deterministic part.  src/utils/sampling.cu:139-142 (sf), :241-291 (penalty, temperature
// in base-2 units, softmax), :294-362 (threshold search on float bit patterns), :365-404 (tie
// compensation), :461-470 (penalty update), argument normalisation :507-512 and
// log2_inv_temp = log2(e)/temperature :526.
// ---------------------------------------------------------------------------------------------
static inline float sf(float x) {
  const float y = std::isnan(x) ? 0.0f : x;
  return std::isinf(y) ? std::copysign(3.402823466e+38f, y) : y;
}

static void sampler_probs(int V, const float* logits, const float* penalties, float temperature, float* probs) {
  const float log2_inv_temp = static_cast<float>(1.44269504088896340736 / static_cast<double>(temperature));
  float maxu = -INFINITY;
  for (int i = 0; i < V; ++i) {
    const float pen = penalties ? penalties[i] : 0.0f;
    probs[i] = sf((sf(logits[i]) - pen) * log2_inv_temp);
    maxu = std::max(maxu, probs[i]);
  }
  float denom = 0.0f;
  for (int i = 0; i < V; ++i) denom += std::exp2(probs[i] - maxu);
  for (int i = 0; i < V; ++i) probs[i] = std::exp2(probs[i] - maxu) / denom;
}

int orc_sample_greedy_penalty(int V, const float* logits, float* penalties, float presence, float frequency,
                              float decay, float temperature) {
  const float log2_inv_temp = static_cast<float>(1.44269504088896340736 / static_cast<double>(temperature));
  int best = 0;
  float bestv = -INFINITY;
  for (int i = 0; i < V; ++i) {
    const float u = sf((sf(logits[i]) - penalties[i]) * log2_inv_temp);
    if (u > bestv) {
      bestv = u;
      best = i;
    }
  }
  for (int i = 0; i < V; ++i) {
    const float p = penalties[i];
    penalties[i] = p * decay + ((i != best) ? 0.0f : (p == 0.0f ? presence : frequency));
  }
  return best;
}

int orc_sample_filter(int V, const float* logits, const float* penalties, float temperature, int top_k,
                      float top_p, float* probs) {
  if (top_k <= 0 || top_k > V) top_k = V;
  if (top_p < 0.0f || top_p > 1.0f) top_p = 1.0f;
  if (top_p == 0.0f) {
    top_k = 1;
    top_p = 1.0f;
  }
  sampler_probs(V, logits, penalties, temperature, probs);
  float pmax = -INFINITY, pmin = INFINITY;
  for (int i = 0; i < V; ++i) {
    pmax = std::max(pmax, probs[i]);
    pmin = std::min(pmin, probs[i]);
  }
  auto bits = [](float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
  };
  auto unbits = [](uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
  };
  auto count_mass = [&](uint32_t pivot, unsigned& cnt, float& mass) {
    const float t = unbits(pivot);
    cnt = 0;
    double m = 0.0;
    for (int i = 0; i < V; ++i)
      if (probs[i] >= t) {
        ++cnt;
        m += probs[i];
      }
    mass = static_cast<float>(m);
  };
  uint32_t left = bits(pmin), right = bits(pmax) + 1;
  unsigned cnt = static_cast<unsigned>(V);
  float mass = 1.0f;
  while ((cnt > static_cast<unsigned>(top_k) || mass > top_p) && left < right - 1) {
    const uint32_t mid = left + (right - left) / 2;
    unsigned c;
    float m;
    count_mass(mid, c, m);
    if (c < static_cast<unsigned>(top_k) && m < top_p) {
      right = mid;
    } else {
      left = mid;
      cnt = c;
      mass = m;
    }
  }
  const float thr = unbits(left);
  unsigned eqk = 0, gtk = 0;
  double gtp = 0.0;
  for (int i = 0; i < V; ++i) {
    if (probs[i] == thr) ++eqk;
    if (probs[i] > thr) {
      ++gtk;
      gtp += probs[i];
    }
  }
  float comp = 1.0f;
  if (eqk > 0) {
    comp = std::min(sf((top_p - static_cast<float>(gtp)) / (thr * eqk)), comp);
    comp = std::min(sf(static_cast<float>(top_k - static_cast<int>(gtk)) / eqk), comp);
    comp = std::max(comp, 0.0f);
  }
  int kept = 0;
  for (int i = 0; i < V; ++i) {
    const float p = probs[i];
    probs[i] = (p < thr) ? 0.0f : (p == thr ? p * comp : p);
    if (probs[i] > 0.0f) ++kept;
  }
  return kept;
}

// ---------------------------------------------------------------------------------------------
// Model graph: src/rwkv7_fast_v4.cu:1046-1345 (run_backend_forward).  Order of ops, layer-0
// special cases (v_first, no v LoRA: :1171,1246-1247), state slices (:1177-1185), last-token
// logits (:1314-1342).  Rounding points are those of the reference's fused decode path (the
// fused LoRA-out kernels keep tanh/sigmoid/v12 in fp32, cuda/rwkv7_v3a_ops.cu:1082-1123), used
// here for every shape.  ffn.value is kept [C,F] ("out,in") and accumulated in fp32 (the
// reference's dense path, src/rwkv7_fast_v4.cu:1294-1295).
// ---------------------------------------------------------------------------------------------
struct OrcMatrix {
  int fmt = ORC_FMT_F16;
  const void* data = nullptr;
  const uint16_t* scale = nullptr;
  const uint8_t* zp = nullptr;
};

struct OrcLayer {
  const uint16_t* t[64] = {nullptr};
  OrcMatrix m[6];
};

struct OrcModel {
  int L, C, H, F, V, Rw, Ra, Rg, Rv;
  const uint16_t* emb_ln0 = nullptr;
  const uint16_t* ln_out_w = nullptr;
  const uint16_t* ln_out_b = nullptr;
  OrcMatrix head;
  std::vector<OrcLayer> layers;
};

OrcModel* orc_model_create(int L, int C, int H, int F, int V, int Rw, int Ra, int Rg, int Rv) {
  if (L <= 0 || C != H * kHead || F <= 0 || V <= 0) return nullptr;
  OrcModel* m = new OrcModel();
  m->L = L; m->C = C; m->H = H; m->F = F; m->V = V;
  m->Rw = Rw; m->Ra = Ra; m->Rg = Rg; m->Rv = Rv;
  m->layers.resize(L);
  return m;
}

void orc_model_destroy(OrcModel* m) { delete m; }

int orc_model_set_tensor(OrcModel* m, int layer, int id, const uint16_t* data) {
  if (layer < 0) {
    if (id == ORC_T_EMB_LN0) m->emb_ln0 = data;
    else if (id == ORC_T_LN_OUT_W) m->ln_out_w = data;
    else if (id == ORC_T_LN_OUT_B) m->ln_out_b = data;
    else return -1;
    return 0;
  }
  if (layer >= m->L || id < 0 || id >= 64) return -1;
  m->layers[layer].t[id] = data;
  return 0;
}

int orc_model_set_matrix(OrcModel* m, int layer, int id, int fmt, const void* data, const uint16_t* scale,
                         const uint8_t* zp) {
  OrcMatrix mat;
  mat.fmt = fmt; mat.data = data; mat.scale = scale; mat.zp = zp;
  if (id == ORC_M_HEAD) {
    m->head = mat;
    return 0;
  }
  if (layer < 0 || layer >= m->L || id < 0 || id >= 6) return -1;
  m->layers[layer].m[id] = mat;
  return 0;
}

static void mat_apply(const OrcMatrix& mat, int M, int N, int K, const uint16_t* x, uint16_t* y) {
  gemv_any_f16(mat.fmt, M, N, K, x, mat.data, mat.scale, mat.zp, y);
}

static int model_forward_impl(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift, float* wkv,
                              uint16_t* wkv16, int32_t* elapsed, float* logits, uint16_t* trace);

int orc_model_forward(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift, float* wkv,
                      int32_t* elapsed, float* logits, uint16_t* trace) {
  return model_forward_impl(m, tokens, B, T, shift, wkv, nullptr, elapsed, logits, trace);
}

// The same graph with the WKV state in fp16 (ModelBackend's use_wkv32 == false, src/rwkv7_fast_v4.cu:1266-1271):
// calls of up to 16 tokens add w0 to the decay logit inside the recurrence, unrounded; longer ones round
// w12 + w0 to fp16 first (rwkv7_add_vec_launch), as the fp32 path always does.
int orc_model_forward_f16state(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift,
                               uint16_t* wkv16, int32_t* elapsed, float* logits, uint16_t* trace) {
  if (!wkv16) return -1;
  return model_forward_impl(m, tokens, B, T, shift, nullptr, wkv16, elapsed, logits, trace);
}

static int model_forward_impl(const OrcModel* m, const int64_t* tokens, int B, int T, uint16_t* shift, float* wkv,
                              uint16_t* wkv16, int32_t* elapsed, float* logits, uint16_t* trace) {
  if (!m || B <= 0 || T <= 0) return -1;
  const int C = m->C, H = m->H, F = m->F, V = m->V, L = m->L;
  const int rows = B * T;
  const int64_t RC = static_cast<int64_t>(rows) * C;
  for (int i = 0; i < rows; ++i)
    if (tokens[i] < 0 || tokens[i] >= V) return -2;  // src/rwkv7_fast_v4.cu:1107-1110

  std::vector<uint16_t> x(RC), xx(RC), xr(RC), xw(RC), xk(RC), xv(RC), xa(RC), xg(RC), r(RC), k(RC), v(RC),
      v_first(RC), w12(RC), a12(RC), g(RC), k2(RC), nkk(RC), kka(RC), w_raw(RC), y(RC), y2(RC), att(RC), x1(RC),
      ln2(RC), mixed(RC), cm(RC), hid(static_cast<size_t>(rows) * F), act(static_cast<size_t>(rows) * F),
      xf(static_cast<size_t>(B) * C);
  std::vector<float> tmp32(RC);

  for (int i = 0; i < rows; ++i)
    std::memcpy(&x[static_cast<int64_t>(i) * C], m->emb_ln0 + tokens[i] * C, sizeof(uint16_t) * C);
  orc_layer_norm(rows, C, x.data(), m->layers[0].t[ORC_T_LN1_W], m->layers[0].t[ORC_T_LN1_B], xx.data(), 1e-5f);

  for (int l = 0; l < L; ++l) {
    const OrcLayer& w = m->layers[l];
    uint16_t* shift0 = shift + static_cast<int64_t>(l) * 2 * B * C;
    uint16_t* shift1 = shift0 + static_cast<int64_t>(B) * C;
    float* S = wkv ? wkv + static_cast<int64_t>(l) * B * H * kHead * kHead : nullptr;
    uint16_t* S16 = wkv16 ? wkv16 + static_cast<int64_t>(l) * B * H * kHead * kHead : nullptr;

    const uint16_t* mu6[6] = {w.t[ORC_T_X_R], w.t[ORC_T_X_W], w.t[ORC_T_X_K], w.t[ORC_T_X_V], w.t[ORC_T_X_A], w.t[ORC_T_X_G]};
    uint16_t* out6[6] = {xr.data(), xw.data(), xk.data(), xv.data(), xa.data(), xg.data()};
    orc_token_shift_mix(B, T, C, 6, xx.data(), shift0, mu6, out6);

    mat_apply(w.m[ORC_M_ATT_R], rows, C, C, xr.data(), r.data());
    mat_apply(w.m[ORC_M_ATT_K], rows, C, C, xk.data(), k.data());
    mat_apply(w.m[ORC_M_ATT_V], rows, C, C, xv.data(), v.data());

    orc_lora(rows, C, m->Rw, 1, xw.data(), w.t[ORC_T_W1], w.t[ORC_T_W2], tmp32.data());
    orc_f32_to_f16_array(tmp32.data(), w12.data(), RC);
    orc_lora(rows, C, m->Ra, 0, xa.data(), w.t[ORC_T_A1], w.t[ORC_T_A2], tmp32.data());
    orc_f32_to_f16_array(tmp32.data(), a12.data(), RC);
    orc_lora(rows, C, m->Rg, 2, xg.data(), w.t[ORC_T_G1], w.t[ORC_T_G2], tmp32.data());
    orc_f32_to_f16_array(tmp32.data(), g.data(), RC);
    if (l == 0) {
      v_first = v;
    } else {
      orc_lora(rows, C, m->Rv, 0, xv.data(), w.t[ORC_T_V1], w.t[ORC_T_V2], tmp32.data());
      std::vector<uint16_t> vout(RC);
      orc_vres_gate(rows, C, v.data(), v_first.data(), w.t[ORC_T_V0], tmp32.data(), vout.data());
      v.swap(vout);
    }

    orc_kk_a_gate(rows, C, H, k.data(), w.t[ORC_T_K_K], w.t[ORC_T_A0], a12.data(), w.t[ORC_T_K_A], k2.data(),
                  nkk.data(), kka.data());
    if (S16 && T <= 16) {
      orc_wkv7_f16state(B, T, C, H, S16, r.data(), w12.data(), w.t[ORC_T_W0], k2.data(), v.data(), nkk.data(), kka.data(),
                        y.data(), elapsed);
    } else {
      orc_add_vec(rows, C, w12.data(), w.t[ORC_T_W0], w_raw.data());
      if (S16) {
        orc_wkv7_f16state(B, T, C, H, S16, r.data(), w_raw.data(), nullptr, k2.data(), v.data(), nkk.data(), kka.data(),
                          y.data(), elapsed);
      } else {
        orc_wkv7_f16(B, T, C, H, 0, S, r.data(), w_raw.data(), k2.data(), v.data(), nkk.data(), kka.data(), y.data());
      }
    }
    orc_lnx_rkvres_xg(rows, C, H, y.data(), r.data(), k2.data(), v.data(), w.t[ORC_T_R_K], w.t[ORC_T_LNX_W],
                      w.t[ORC_T_LNX_B], g.data(), y2.data());
    mat_apply(w.m[ORC_M_ATT_O], rows, C, C, y2.data(), att.data());

    orc_add_layer_norm(rows, C, x.data(), att.data(), w.t[ORC_T_LN2_W], w.t[ORC_T_LN2_B], x1.data(), ln2.data(), 1e-5f);
    const uint16_t* mu1[1] = {w.t[ORC_T_FFN_X_K]};
    uint16_t* out1[1] = {mixed.data()};
    orc_token_shift_mix(B, T, C, 1, ln2.data(), shift1, mu1, out1);

    mat_apply(w.m[ORC_M_FFN_KEY], rows, F, C, mixed.data(), hid.data());
    orc_relu_square(static_cast<int64_t>(rows) * F, hid.data(), act.data());
    mat_apply(w.m[ORC_M_FFN_VALUE], rows, C, F, act.data(), cm.data());

    if (l + 1 < L) {
      const OrcLayer& nx = m->layers[l + 1];
      std::vector<uint16_t> xn(RC);
      orc_add_layer_norm(rows, C, x1.data(), cm.data(), nx.t[ORC_T_LN1_W], nx.t[ORC_T_LN1_B], xn.data(), xx.data(), 1e-5f);
      x.swap(xn);
    } else {
      orc_add_last_layer_norm(B, T, C, x1.data(), cm.data(), m->ln_out_w, m->ln_out_b, xf.data(), 1e-5f);
      for (int64_t i = 0; i < RC; ++i) x[i] = f2h(h2f(x1[i]) + h2f(cm[i]));
    }
    if (trace) std::memcpy(trace + static_cast<int64_t>(l) * RC, x.data(), sizeof(uint16_t) * RC);
  }

  for (int b = 0; b < B; ++b) elapsed[b] += T;  // cuda/rwkv7_v3a_ops.cu:202-207
  // head GEMV -> fp16 -> fp32 (src/rwkv7_fast_v4.cu:1325-1341)
  std::vector<uint16_t> l16(static_cast<size_t>(B) * V);
  mat_apply(m->head, B, V, C, xf.data(), l16.data());
  orc_f16_to_f32_array(l16.data(), logits, static_cast<int64_t>(B) * V);
  return 0;
}
