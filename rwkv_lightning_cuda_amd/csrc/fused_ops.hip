// Fused element-wise / normalisation kernels of the RWKV-7 layer graph.
//
// Reference kernels restated here (same arithmetic and fp16 rounding points, re-tiled for wave64):
//   LayerNorm family ........ cuda/rwkv7_v3a_ops.cu:1272-1351 (LN, add+LN), :1800-1931 (add + last-token LN),
//                             :1933-1985 (add+LN+cmix lerp), :1987-2060 (add+LN+6 lerps)
//   token shift ............. cuda/rwkv7_fast_ops_fp16.cu:53-127 (mix6 + shift update), :393-419 (cmix mix)
//   kk / a-gate ............. cuda/rwkv7_fast_ops_fp16.cu:129-172
//   GroupNorm+rkv-res+gate .. cuda/rwkv7_fast_ops_fp16.cu:174-237
//   relu^2, add_vec, f16->f32 cuda/rwkv7_fast_ops_fp16.cu:421-485;  advance_i32 cuda/rwkv7_v3a_ops.cu:202-207
//
// The LN kernels keep the whole row in registers (one block per row, one 16-byte slice per thread: 256, 512 or
// 1024 threads by row length - decode steps have few rows, so the wavefronts of a row are the only parallelism the
// launch has: 512 threads instead of 256 with two slices each make a 4096-wide row 15-25 % faster), so a row is
// read from HBM once for the two-pass mean/variance and the normalise+lerp epilogue.
#include "ops.h"

namespace rwkv {

constexpr int kLnMaxThreads = 1024;  // one 8-element vector per thread -> C <= 8192



template <int MODE, int NT>
__global__ __launch_bounds__(NT) void ln_fused_kernel(LnArgs a) {
  constexpr int kLnThreads = NT;
  constexpr int kLnMaxVec = 1;
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const int C = a.C;
  int64_t src = static_cast<int64_t>(row) * C;
  if constexpr (MODE == kAddLastLn) src = (static_cast<int64_t>(row) * a.T + (a.T - 1)) * C;
  int64_t xsrc = src;
  if constexpr (MODE == kLnMix) {
    if (a.tokens) xsrc = a.tokens[row] * static_cast<int64_t>(C);
  }
  const int64_t dst = static_cast<int64_t>(row) * C;

  // every global load of the kernel is issued here, before the first reduction, so the block pays one
  // memory round trip instead of three
  float v[kLnMaxVec][8];
  half8_t wv[kLnMaxVec], bv[kLnMaxVec], pv[kLnMaxVec], mv[kLnMaxVec][6];
  constexpr bool kMix = (MODE == kAddLnMix || MODE == kLnMix);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < kLnMaxVec; ++i) {
    const int c = (i * kLnThreads + threadIdx.x) * 8;
    if (c < C) {
      // the parameter vectors first: the sum over split-K partials below waits for its loads, and loads return in
      // issue order, so anything requested after that loop would cost a second trip to memory
      wv[i] = *reinterpret_cast<const half8_t*>(a.w + c);
      bv[i] = *reinterpret_cast<const half8_t*>(a.b + c);
      if constexpr (kMix) {
        pv[i] = *reinterpret_cast<const half8_t*>(a.shift + dst + c);
        // (no branch per coefficient vector: the unused ones re-read the last one, which costs nothing, whereas a
        // load under a branch is followed by a wait for everything requested so far)
#pragma unroll
        for (int s = 0; s < 6; ++s) mv[i][s] = *reinterpret_cast<const half8_t*>(a.mu[s < a.n_mix ? s : a.n_mix - 1] + c);
      }
      const half8_t xv = *reinterpret_cast<const half8_t*>(a.x + xsrc + c);
      __builtin_amdgcn_sched_barrier(0);
      half8_t rv = {};
      if constexpr (MODE != kLn && MODE != kLnMix) {
        if (a.res_partial) {
          // (the scale vector before the partials, for the same reason; without one any valid vector is read)
          const half8_t sv8 = *reinterpret_cast<const half8_t*>((a.res_scale ? a.res_scale : a.w) + c);
          const float* pp = a.res_partial + src + c;
          float4_t s0 = *reinterpret_cast<const float4_t*>(pp);
          float4_t s1 = *reinterpret_cast<const float4_t*>(pp + 4);
          // The other partials four at a time, all requested before the first is added (in split order, as
          // always); past the last split the last one is read again and left out.  A plain loop over the splits
          // would wait for each partial before it asks for the next: one trip to memory per split.
          for (int base = 1; base < a.res_splits; base += 4) {
            float4_t q0[4], q1[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int sp = base + u < a.res_splits ? base + u : a.res_splits - 1;
              q0[u] = *reinterpret_cast<const float4_t*>(pp + sp * a.res_plane);
              q1[u] = *reinterpret_cast<const float4_t*>(pp + sp * a.res_plane + 4);
            }
            // (keeps the four requests together: their only uses sit under the conditions below, and the compiler
            // would move each load down into its condition)
#pragma unroll
            for (int u = 0; u < 4; ++u) asm volatile("" : "+v"(q0[u]), "+v"(q1[u]));
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              if (base + u < a.res_splits) {
                s0 = s0 + q0[u];
                s1 = s1 + q1[u];
              }
            }
          }
          float scl[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) scl[e] = a.res_scale ? h2f(sv8[e]) : 1.0f;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            rv[e] = f2h(mul_f32(s0[e], scl[e]));
            rv[4 + e] = f2h(mul_f32(s1[e], scl[4 + e]));
          }
        } else {
          rv = *reinterpret_cast<const half8_t*>(a.res + src + c);
        }
      }
      if constexpr (MODE == kLn || MODE == kLnMix) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = h2f(xv[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[i][e] = h2f(xv[e]) + h2f(rv[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) sum += v[i][e];
    }
  }
  sum = block_sum<NT / 64>(sum, red);
  const float mean = sum / static_cast<float>(C);
  float sv = 0.0f;
#pragma unroll
  for (int i = 0; i < kLnMaxVec; ++i) {
    const int c = (i * kLnThreads + threadIdx.x) * 8;
    if (c < C) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[i][e] - mean;
        sv = fmaf(d, d, sv);
      }
    }
  }
  sv = block_sum<NT / 64>(sv, red);
  const float rstd = rsqrtf(sv / static_cast<float>(C) + a.eps);

#pragma unroll
  for (int i = 0; i < kLnMaxVec; ++i) {
    const int c = (i * kLnThreads + threadIdx.x) * 8;
    if (c < C) {
      half8_t yv;
#pragma unroll
      for (int e = 0; e < 8; ++e) yv[e] = f2h(fmaf((v[i][e] - mean) * rstd, h2f(wv[i][e]), h2f(bv[i][e])));
      if constexpr (MODE == kAddLn || MODE == kAddLnMix) {
        half8_t xo;
#pragma unroll
        for (int e = 0; e < 8; ++e) xo[e] = f2h(v[i][e]);
        *reinterpret_cast<half8_t*>(a.x_out + dst + c) = xo;
      }
      if constexpr (MODE == kLnMix) {
        if (a.x_out) {  // the residual stream starts as the (already fp16) embedding row
          half8_t xo;
#pragma unroll
          for (int e = 0; e < 8; ++e) xo[e] = f2h(v[i][e]);
          *reinterpret_cast<half8_t*>(a.x_out + dst + c) = xo;
        }
      }
      if constexpr (kMix) {
        // lerps read the fp16-rounded LN output (rwkv7_v3a_ops.cu:1978-1983)
#pragma unroll
        for (int s = 0; s < 6; ++s) {
          if (s < a.n_mix) {
            half8_t ov;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const float yf = h2f(yv[e]);
              ov[e] = f2h(fmaf(h2f(pv[i][e]) - yf, h2f(mv[i][s][e]), yf));
            }
            *reinterpret_cast<half8_t*>(a.out[s] + dst + c) = ov;
          }
        }
        *reinterpret_cast<half8_t*>(a.shift + dst + c) = yv;
        if (a.y) *reinterpret_cast<half8_t*>(a.y + dst + c) = yv;
      } else {
        *reinterpret_cast<half8_t*>(a.y + dst + c) = yv;
      }
    }
  }
}

// ---- residual add + LayerNorm + token shift over sequences (prefill chunks): one block per row (b, t) ----------
// The lerps of row t need the LayerNorm output of row t - 1, which another block computes: instead of a launch of
// its own between the two (the LN rows written and read back, 5 us of launch and ramp), the block normalises the
// previous row a second time - the same loads, the same arithmetic in the same order, so bitwise the value the
// previous row's block gets.  At t == 0 the previous output is the shift row of the state.  Blocks of other rows
// read that shift row while this launch runs, so the new one (the LN output at t == T - 1) goes to shift_next and
// the caller moves it over afterwards.
template <int NT>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* scratch) {  // block_sum's order, two values
  a = wave_sum_dpp(a);
  b = wave_sum_dpp(b);
  if constexpr (NT / 64 == 1) return;
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    scratch[wave] = a;
    scratch[NT / 64 + wave] = b;
  }
  __syncthreads();
  float ta = 0.0f, tb = 0.0f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) {
    ta += scratch[i];
    tb += scratch[NT / 64 + i];
  }
  a = ta;
  b = tb;
}

template <int NT>
__global__ __launch_bounds__(NT) void ln_mix_seq_kernel(LnArgs a) {
  __shared__ float red[2 * (NT / 64)];
  const int row = blockIdx.x;
  const int C = a.C;
  const int bi = row / a.T;
  const int t = row - bi * a.T;
  const bool live = static_cast<int>(threadIdx.x) * 8 < C;
  const int c = live ? threadIdx.x * 8 : 0;  // idle threads repeat slice 0 and store nothing
  const int64_t o = static_cast<int64_t>(row) * C + c;
  const int64_t op = t > 0 ? o - C : o;  // the previous row; at t == 0 this row again, unused

  // every load of the kernel up front, none under a per-lane branch
  const half8_t wv = *reinterpret_cast<const half8_t*>(a.w + c);
  const half8_t bv = *reinterpret_cast<const half8_t*>(a.b + c);
  const half8_t sh = *reinterpret_cast<const half8_t*>(a.shift + static_cast<int64_t>(bi) * C + c);
  half8_t mv[6];
#pragma unroll
  for (int s = 0; s < 6; ++s) mv[s] = *reinterpret_cast<const half8_t*>(a.mu[s < a.n_mix ? s : a.n_mix - 1] + c);
  const half8_t xv = *reinterpret_cast<const half8_t*>(a.x + o);
  const half8_t xp = *reinterpret_cast<const half8_t*>(a.x + op);
  half8_t rv, rp;
  if (a.res_partial) {
    const half8_t sv8 = *reinterpret_cast<const half8_t*>((a.res_scale ? a.res_scale : a.w) + c);
    const float* pp = a.res_partial + o;
    const float* pq = a.res_partial + op;
    float4_t s0 = *reinterpret_cast<const float4_t*>(pp), s1 = *reinterpret_cast<const float4_t*>(pp + 4);
    float4_t u0 = *reinterpret_cast<const float4_t*>(pq), u1 = *reinterpret_cast<const float4_t*>(pq + 4);
    // the other partials four at a time, all requested before the first is added, in split order (ln_fused_kernel)
    for (int base = 1; base < a.res_splits; base += 4) {
      float4_t q0[4], q1[4], p0[4], p1[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t sp = (base + u < a.res_splits ? base + u : a.res_splits - 1) * a.res_plane;
        q0[u] = *reinterpret_cast<const float4_t*>(pp + sp);
        q1[u] = *reinterpret_cast<const float4_t*>(pp + sp + 4);
        p0[u] = *reinterpret_cast<const float4_t*>(pq + sp);
        p1[u] = *reinterpret_cast<const float4_t*>(pq + sp + 4);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) asm volatile("" : "+v"(q0[u]), "+v"(q1[u]), "+v"(p0[u]), "+v"(p1[u]));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (base + u < a.res_splits) {
          s0 = s0 + q0[u]; s1 = s1 + q1[u];
          u0 = u0 + p0[u]; u1 = u1 + p1[u];
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float sl = a.res_scale ? h2f(sv8[e]) : 1.0f, sh4 = a.res_scale ? h2f(sv8[4 + e]) : 1.0f;
      rv[e] = f2h(mul_f32(s0[e], sl)); rv[4 + e] = f2h(mul_f32(s1[e], sh4));
      rp[e] = f2h(mul_f32(u0[e], sl)); rp[4 + e] = f2h(mul_f32(u1[e], sh4));
    }
  } else {
    rv = *reinterpret_cast<const half8_t*>(a.res + o);
    rp = *reinterpret_cast<const half8_t*>(a.res + op);
  }

  float v[8], vp[8];
  float sum = 0.0f, sump = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    v[e] = h2f(xv[e]) + h2f(rv[e]);
    vp[e] = h2f(xp[e]) + h2f(rp[e]);
    if (!live) v[e] = vp[e] = 0.0f;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) sum += v[e];
#pragma unroll
  for (int e = 0; e < 8; ++e) sump += vp[e];
  block_sum2<NT>(sum, sump, red);
  const float mean = sum / static_cast<float>(C), meanp = sump / static_cast<float>(C);
  float sv = 0.0f, svp = 0.0f;
  if (live) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = v[e] - mean;
      sv = fmaf(d, d, sv);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = vp[e] - meanp;
      svp = fmaf(d, d, svp);
    }
  }
  block_sum2<NT>(sv, svp, red);
  const float rstd = rsqrtf(sv / static_cast<float>(C) + a.eps);
  const float rstdp = rsqrtf(svp / static_cast<float>(C) + a.eps);
  if (!live) return;

  half8_t yv, xo;
  float prev[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // Both outputs as an fp32 fma rounded to fp16 afterwards (what the LayerNorm kernels store).  Left alone, the
    // compiler folds the conversion of the one that is not stored into the fma (v_fma_mixlo_f16: one rounding
    // instead of two), and the previous row's value then differs from what that row's own block gets in one
    // element of some ten thousand.  The same for the lerps below, against token_shift_mix_kernel.
    yv[e] = f2h_apart(fmaf((v[e] - mean) * rstd, h2f(wv[e]), h2f(bv[e])));
    const half_t yp = f2h_apart(fmaf((vp[e] - meanp) * rstdp, h2f(wv[e]), h2f(bv[e])));
    prev[e] = t > 0 ? h2f(yp) : h2f(sh[e]);
    xo[e] = f2h(v[e]);
  }
  *reinterpret_cast<half8_t*>(a.x_out + o) = xo;
  // lerps read the fp16-rounded LN output (rwkv7_v3a_ops.cu:1978-1983)
#pragma unroll
  for (int s = 0; s < 6; ++s) {
    if (s < a.n_mix) {
      half8_t ov;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float yf = h2f(yv[e]);
        ov[e] = f2h_apart(fmaf(prev[e] - yf, h2f(mv[s][e]), yf));
      }
      *reinterpret_cast<half8_t*>(a.out[s] + o) = ov;
    }
  }
  if (a.y) *reinterpret_cast<half8_t*>(a.y + o) = yv;
  if (t == a.T - 1) *reinterpret_cast<half8_t*>(a.shift_next + static_cast<int64_t>(bi) * C + c) = yv;
}

static int check_ln_shape(int rows, int C) {
  RWKV_REQUIRE(rows > 0, "layer norm: rows must be positive");
  RWKV_REQUIRE(C > 0 && C % 8 == 0 && C <= kLnMaxThreads * 8,
               "layer norm: C (%d) must be a multiple of 8 and at most %d", C, kLnMaxThreads * 8);
  return RWKV_OK;
}

template <int NT>
static int ln_launch_nt(hipStream_t st, int mode, int rows, const LnArgs& a) {
  switch (mode) {
    case kLn: hipLaunchKernelGGL((ln_fused_kernel<kLn, NT>), dim3(rows), dim3(NT), 0, st, a); break;
    case kAddLn: hipLaunchKernelGGL((ln_fused_kernel<kAddLn, NT>), dim3(rows), dim3(NT), 0, st, a); break;
    case kAddLastLn: hipLaunchKernelGGL((ln_fused_kernel<kAddLastLn, NT>), dim3(rows), dim3(NT), 0, st, a); break;
    case kAddLnMix: hipLaunchKernelGGL((ln_fused_kernel<kAddLnMix, NT>), dim3(rows), dim3(NT), 0, st, a); break;
    case kLnMix: hipLaunchKernelGGL((ln_fused_kernel<kLnMix, NT>), dim3(rows), dim3(NT), 0, st, a); break;
    default: set_error("bad layer-norm mode %d", mode); return RWKV_E_INVALID;
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int ln_launch(hipStream_t st, int mode, int rows, const LnArgs& a) {
  if (int rc = check_ln_shape(rows, a.C)) return rc;
  if (mode == kAddLnMixSeq) {
    RWKV_REQUIRE(a.C <= 512 * 8, "layer norm + token shift over a sequence: C (%d) must be at most 4096", a.C);
    RWKV_REQUIRE(a.T >= 1 && rows % a.T == 0 && a.shift && a.shift_next && a.x_out && a.n_mix >= 1 && a.n_mix <= 6 &&
                     (a.res || a.res_partial),
                 "layer norm + token shift over a sequence: bad arguments");
    // the block of row t reads x and the residual of row t - 1 again while that row's block stores its outputs:
    // no output may share memory with an input
    RWKV_REQUIRE(a.x_out != a.x && a.y != a.x && (a.res == nullptr || (a.x_out != a.res && a.y != a.res)),
                 "layer norm + token shift over a sequence: outputs must not alias x or the residual");
    if (a.C <= 256 * 8) hipLaunchKernelGGL(ln_mix_seq_kernel<256>, dim3(rows), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(ln_mix_seq_kernel<512>, dim3(rows), dim3(512), 0, st, a);
    RWKV_LAUNCH_CHECK();
    return RWKV_OK;
  }
  if (a.C <= 256 * 8) return ln_launch_nt<256>(st, mode, rows, a);
  if (a.C <= 512 * 8) return ln_launch_nt<512>(st, mode, rows, a);
  return ln_launch_nt<1024>(st, mode, rows, a);
}

// ---- token shift: out_s = x + (prev - x) * mu_s with prev = shift[b] at t == 0, else x[b,t-1];
// then shift[b] = x[b,T-1].  One thread per (row, 8 channels); the thread of token 0 reads the old shift slice
// and then overwrites it, so no thread can overwrite a slice another one still has to read. ------------

__global__ __launch_bounds__(256) void token_shift_mix_kernel(MixArgs a) {
  const int cvecs = a.C / 8;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= static_cast<int64_t>(a.B) * a.T * cvecs) return;
  const int64_t row = idx / cvecs;
  const int c = static_cast<int>(idx - row * cvecs) * 8;
  const int b = static_cast<int>(row / a.T);
  const int t = static_cast<int>(row - static_cast<int64_t>(b) * a.T);
  const int64_t o = row * a.C + c;
  const half8_t cur = *reinterpret_cast<const half8_t*>(a.x + o);
  const half8_t prev = (t == 0) ? *reinterpret_cast<const half8_t*>(a.shift + static_cast<int64_t>(b) * a.C + c)
                                : *reinterpret_cast<const half8_t*>(a.x + o - a.C);
  for (int s = 0; s < a.n_mix; ++s) {
    const half8_t mu = *reinterpret_cast<const half8_t*>(a.mu[s] + c);
    half8_t ov;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float cf = h2f(cur[e]);
      ov[e] = f2h(cf + (h2f(prev[e]) - cf) * h2f(mu[e]));
    }
    *reinterpret_cast<half8_t*>(a.out[s] + o) = ov;
  }
  // the thread that read the old shift slice replaces it with the last token's slice: no other thread touches it
  if (t == 0) {
    const half8_t last = (a.T == 1) ? cur : *reinterpret_cast<const half8_t*>(a.x + o + static_cast<int64_t>(a.T - 1) * a.C);
    *reinterpret_cast<half8_t*>(a.shift + static_cast<int64_t>(b) * a.C + c) = last;
  }
}

int token_shift_mix_launch(hipStream_t st, const MixArgs& a) {
  RWKV_REQUIRE(a.B > 0 && a.T > 0 && a.C > 0 && a.C % 8 == 0, "token shift: bad shape B=%d T=%d C=%d", a.B, a.T, a.C);
  RWKV_REQUIRE(a.n_mix >= 1 && a.n_mix <= 6, "token shift: n_mix %d out of range", a.n_mix);
  const int64_t n = static_cast<int64_t>(a.B) * a.T * (a.C / 8);
  hipLaunchKernelGGL(token_shift_mix_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, st, a);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// ---- kk normalise + a-gate: one wave per (row, head), lane = channel --------------------------------
// Optional fp32 outputs feed the WKV sequence kernel directly (values are the fp16-rounded ones).

__global__ __launch_bounds__(256) void kk_a_gate_kernel(KkArgs p) {
  const int64_t rh = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (rh >= p.rows_heads) return;
  const int lane = threadIdx.x & 63;
  const int h = static_cast<int>(rh % p.H);
  const int64_t idx = rh * kHead + lane;
  const int c = h * kHead + lane;
  const float kv = h2f(p.k[idx]);
  const float u = kv * h2f(p.k_k[c]);
  const float total = wave_sum(u * u);
  const float inv = 1.0f / fmaxf(sqrtf(total), kKkEps);
  const float kk = u * inv;
  const float av = sigmoid_f(h2f(p.a0[c]) + h2f(p.a12[idx]));
  const float ka = h2f(p.k_a[c]);
  const half_t nk = f2h(kv * fmaf(av, ka, 1.0f - ka));
  const half_t nkk = f2h(-kk);
  const half_t kka = f2h(kk * av);
  if (p.new_k) p.new_k[idx] = nk;
  if (p.neg_kk) p.neg_kk[idx] = nkk;
  if (p.kka) p.kka[idx] = kka;
  if (p.k32) {
    p.k32[idx] = h2f(nk);
    p.a32[idx] = h2f(nkk);
    p.b32[idx] = h2f(kka);
    const float wraw = round_h(h2f(p.w12[idx]) + h2f(p.w0[c]));  // rwkv7_add_vec_launch rounding point
    p.d32[idx] = exp2f(-0.8750387749145276f / (1.0f + exp2f(-1.4426950408889634f * wraw)));
    p.r32[idx] = h2f(p.r[idx]);
  }
  if (p.w_sum16) p.w_sum16[idx] = f2h(h2f(p.w12[idx]) + h2f(p.w0[c]));
}

int kk_a_gate_launch(hipStream_t st, const KkArgs& p) {
  RWKV_REQUIRE(p.rows_heads > 0 && p.H > 0, "kk_a_gate: bad shape");
  RWKV_REQUIRE(p.w_sum16 == nullptr || (p.w12 && p.w0), "kk_a_gate: the rounded decay logit needs w12 and w0");
  hipLaunchKernelGGL(kk_a_gate_kernel, dim3(ceil_div(p.rows_heads, 4)), dim3(256), 0, st, p);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// ---- per-head GroupNorm + rkv residual + gate: one wave per (row, head) --------------------------------
__global__ __launch_bounds__(256) void lnx_rkvres_xg_kernel(int64_t rows_heads, int H, const half_t* __restrict__ y,
                                                            const half_t* __restrict__ r, const half_t* __restrict__ k,
                                                            const half_t* __restrict__ v, const half_t* __restrict__ r_k,
                                                            const half_t* __restrict__ lnw, const half_t* __restrict__ lnb,
                                                            const half_t* __restrict__ g, half_t* __restrict__ out) {
  const int64_t rh = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (rh >= rows_heads) return;
  const int lane = threadIdx.x & 63;
  const int h = static_cast<int>(rh % H);
  const int64_t idx = rh * kHead + lane;
  const int c = h * kHead + lane;
  const float yv = h2f(y[idx]);
  const float mean = wave_sum(yv) * (1.0f / 64.0f);
  const float d = yv - mean;
  const float var = wave_sum(d * d) * (1.0f / 64.0f);
  const float rstd = rsqrtf(var + kLnxEps);
  const float rkv = wave_sum(h2f(r[idx]) * h2f(k[idx]) * h2f(r_k[c]));
  const float o = (d * rstd * h2f(lnw[c]) + h2f(lnb[c]) + rkv * h2f(v[idx])) * h2f(g[idx]);
  out[idx] = f2h(o);
}

// ---- small element-wise kernels ---------------------------------------------------------------------
__global__ __launch_bounds__(256) void relu_square_kernel(int64_t n, const half_t* __restrict__ x, half_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = fmaxf(h2f(x[i]), 0.0f);
  out[i] = f2h(v * v);
}

__global__ __launch_bounds__(256) void add_vec_kernel(int64_t n, int C, const half_t* __restrict__ x,
                                                      const half_t* __restrict__ vec, half_t* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  out[i] = f2h(h2f(x[i]) + h2f(vec[i % C]));
}

__global__ __launch_bounds__(256) void f16_to_f32_kernel(int64_t n, const half_t* __restrict__ src, float* __restrict__ dst) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= n) return;
  dst[i] = h2f(src[i]);
}

__global__ __launch_bounds__(256) void advance_i32_kernel(int n, int amount, int* __restrict__ x) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] += amount;
}

// gather embedding rows for T > 1: out[row] = table[tokens[row]]
__global__ __launch_bounds__(256) void embed_gather_kernel(int C, const int64_t* __restrict__ tokens,
                                                           const half_t* __restrict__ table, half_t* __restrict__ out) {
  const int row = blockIdx.x;
  const int64_t src = tokens[row] * static_cast<int64_t>(C);
  for (int c = threadIdx.x * 8; c < C; c += 256 * 8)
    *reinterpret_cast<half8_t*>(out + static_cast<int64_t>(row) * C + c) = *reinterpret_cast<const half8_t*>(table + src + c);
}

int embed_gather_launch(hipStream_t st, int rows, int C, const int64_t* tokens, const half_t* table, half_t* out) {
  hipLaunchKernelGGL(embed_gather_kernel, dim3(rows), dim3(256), 0, st, C, tokens, table, out);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int lnx_launch(hipStream_t st, int64_t rows_heads, int H, const half_t* y, const half_t* r, const half_t* k,
               const half_t* v, const half_t* r_k, const half_t* lnw, const half_t* lnb, const half_t* g, half_t* out) {
  hipLaunchKernelGGL(lnx_rkvres_xg_kernel, dim3(ceil_div(rows_heads, 4)), dim3(256), 0, st, rows_heads, H, y, r, k, v,
                     r_k, lnw, lnb, g, out);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int add_vec_launch(hipStream_t st, int rows, int C, const half_t* x, const half_t* vec, half_t* out) {
  const int64_t n = static_cast<int64_t>(rows) * C;
  hipLaunchKernelGGL(add_vec_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, st, n, C, x, vec, out);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int advance_launch(hipStream_t st, int n, int amount, int* x) {
  hipLaunchKernelGGL(advance_i32_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, st, n, amount, x);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

#define H16(p) static_cast<const half_t*>(p)
#define H16M(p) static_cast<half_t*>(p)

extern "C" {

int rwkv_hip_layer_norm(rwkv_stream_t s, int rows, int C, const void* x, const void* w, const void* b, void* y,
                        float eps) {
  RWKV_REQUIRE(x && w && b && y, "layer_norm: NULL tensor");
  LnArgs a = {};
  a.x = H16(x); a.w = H16(w); a.b = H16(b); a.y = H16M(y); a.C = C; a.T = 1; a.eps = eps;
  return ln_launch(as_stream(s), kLn, rows, a);
}

int rwkv_hip_add_layer_norm(rwkv_stream_t s, int rows, int C, const void* x, const void* res, const void* w,
                            const void* b, void* x_out, void* y, float eps) {
  RWKV_REQUIRE(x && res && w && b && x_out && y, "add_layer_norm: NULL tensor");
  LnArgs a = {};
  a.x = H16(x); a.res = H16(res); a.w = H16(w); a.b = H16(b); a.x_out = H16M(x_out); a.y = H16M(y);
  a.C = C; a.T = 1; a.eps = eps;
  return ln_launch(as_stream(s), kAddLn, rows, a);
}

int rwkv_hip_add_last_layer_norm(rwkv_stream_t s, int B, int T, int C, const void* x, const void* res, const void* w,
                                 const void* b, void* y, float eps) {
  RWKV_REQUIRE(x && res && w && b && y && T > 0, "add_last_layer_norm: bad arguments");
  LnArgs a = {};
  a.x = H16(x); a.res = H16(res); a.w = H16(w); a.b = H16(b); a.y = H16M(y); a.C = C; a.T = T; a.eps = eps;
  return ln_launch(as_stream(s), kAddLastLn, B, a);
}

int rwkv_hip_token_shift_mix(rwkv_stream_t s, int B, int T, int C, int n_mix, const void* x, void* shift,
                             const void* const* mu_host, void* const* out_host) {
  RWKV_REQUIRE(x && shift && mu_host && out_host, "token_shift_mix: NULL tensor");
  RWKV_REQUIRE(n_mix >= 1 && n_mix <= 6, "token_shift_mix: n_mix %d out of range", n_mix);
  MixArgs a = {};
  a.x = H16(x); a.shift = H16M(shift); a.B = B; a.T = T; a.C = C; a.n_mix = n_mix;
  for (int i = 0; i < n_mix; ++i) {
    RWKV_REQUIRE(mu_host[i] && out_host[i], "token_shift_mix: NULL tensor");
    a.mu[i] = H16(mu_host[i]);
    a.out[i] = H16M(out_host[i]);
  }
  return token_shift_mix_launch(as_stream(s), a);
}

int rwkv_hip_add_layer_norm_cmix_mix(rwkv_stream_t s, int rows, int C, const void* x, const void* res, void* shift,
                                     const void* w, const void* b, const void* mu_k, void* x_out, void* mixed,
                                     float eps) {
  RWKV_REQUIRE(x && res && shift && w && b && mu_k && x_out && mixed, "add_layer_norm_cmix_mix: NULL tensor");
  LnArgs a = {};
  a.x = H16(x); a.res = H16(res); a.w = H16(w); a.b = H16(b); a.x_out = H16M(x_out); a.shift = H16M(shift);
  a.mu[0] = H16(mu_k); a.out[0] = H16M(mixed); a.n_mix = 1; a.C = C; a.T = 1; a.eps = eps;
  return ln_launch(as_stream(s), kAddLnMix, rows, a);
}

int rwkv_hip_add_layer_norm_tmix_mix6(rwkv_stream_t s, int rows, int C, const void* x, const void* res, void* shift,
                                      const void* w, const void* b, const void* const* mu6_host, void* x_out,
                                      void* const* out6_host, float eps) {
  RWKV_REQUIRE(x && res && shift && w && b && mu6_host && x_out && out6_host, "add_layer_norm_tmix_mix6: NULL tensor");
  LnArgs a = {};
  a.x = H16(x); a.res = H16(res); a.w = H16(w); a.b = H16(b); a.x_out = H16M(x_out); a.shift = H16M(shift);
  for (int i = 0; i < 6; ++i) {
    RWKV_REQUIRE(mu6_host[i] && out6_host[i], "add_layer_norm_tmix_mix6: NULL tensor");
    a.mu[i] = H16(mu6_host[i]);
    a.out[i] = H16M(out6_host[i]);
  }
  a.n_mix = 6; a.C = C; a.T = 1; a.eps = eps;
  return ln_launch(as_stream(s), kAddLnMix, rows, a);
}

int rwkv_hip_kk_a_gate(rwkv_stream_t s, int rows, int C, int H, const void* k, const void* k_k, const void* a0,
                       const void* a12, const void* k_a, void* new_k, void* neg_kk, void* kka) {
  RWKV_REQUIRE(rows > 0 && H > 0 && C == H * kHead, "kk_a_gate: C (%d) must equal H*64", C);
  RWKV_REQUIRE(k && k_k && a0 && a12 && k_a && new_k && neg_kk && kka, "kk_a_gate: NULL tensor");
  KkArgs p = {};
  p.k = H16(k); p.k_k = H16(k_k); p.a0 = H16(a0); p.a12 = H16(a12); p.k_a = H16(k_a);
  p.new_k = H16M(new_k); p.neg_kk = H16M(neg_kk); p.kka = H16M(kka);
  p.rows_heads = static_cast<int64_t>(rows) * H; p.H = H;
  return kk_a_gate_launch(as_stream(s), p);
}

int rwkv_hip_lnx_rkvres_xg(rwkv_stream_t s, int rows, int C, int H, const void* y, const void* r, const void* k,
                           const void* v, const void* r_k, const void* lnw, const void* lnb, const void* g,
                           void* out) {
  RWKV_REQUIRE(rows > 0 && H > 0 && C == H * kHead, "lnx_rkvres_xg: C (%d) must equal H*64", C);
  RWKV_REQUIRE(y && r && k && v && r_k && lnw && lnb && g && out, "lnx_rkvres_xg: NULL tensor");
  return lnx_launch(as_stream(s), static_cast<int64_t>(rows) * H, H, H16(y), H16(r), H16(k), H16(v), H16(r_k),
                    H16(lnw), H16(lnb), H16(g), H16M(out));
}

int rwkv_hip_relu_square(rwkv_stream_t s, int64_t n, const void* x, void* out) {
  RWKV_REQUIRE(n > 0 && x && out, "relu_square: bad arguments");
  hipLaunchKernelGGL(relu_square_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, as_stream(s), n, H16(x), H16M(out));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_add_vec(rwkv_stream_t s, int rows, int C, const void* x, const void* vec, void* out) {
  RWKV_REQUIRE(rows > 0 && C > 0 && x && vec && out, "add_vec: bad arguments");
  return add_vec_launch(as_stream(s), rows, C, H16(x), H16(vec), H16M(out));
}

int rwkv_hip_f16_to_f32(rwkv_stream_t s, int64_t n, const void* src, void* dst) {
  RWKV_REQUIRE(n > 0 && src && dst, "f16_to_f32: bad arguments");
  hipLaunchKernelGGL(f16_to_f32_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, as_stream(s), n, H16(src),
                     static_cast<float*>(dst));
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_advance_i32(rwkv_stream_t s, int n, int amount, void* x) {
  RWKV_REQUIRE(n > 0 && x, "advance_i32: bad arguments");
  return advance_launch(as_stream(s), n, amount, static_cast<int*>(x));
}

}  // extern "C"
