// Sampler: repetition penalty, temperature, softmax, top-k / top-p threshold, inverse-CDF draw, penalty update.
//
// Reference: src/utils/sampling.cu:205-471 (with penalties), :613-848 (without), argument
// normalisation :492-512, sf() :139-142.  Same pipeline and the same threshold definition: the
// largest probability value t (searched by bisection on the IEEE bit pattern, :294-362) such that
// {p >= t} still holds at least top_k entries or at least top_p mass; entries equal to t are scaled by
// `comp` so the kept set has exactly top_k entries / top_p mass (:393-404).
//
// gfx950 re-design: one 1024-thread block (16 wavefronts) per row; each thread owns a fixed set of entries -
// for rows of up to 65536 entries the float4 t, t + 1024, ..., loaded once (coalesced) and kept in registers
// through the softmax, the bisection and the draw; for larger rows a contiguous slice that stays in `probs` -
// so the draw is a single inverse-CDF walk with one uniform number over a fixed order of the row; block
// reductions are wave64 butterflies (DPP and row swaps, no LDS) + one LDS exchange; a bisection step skips the
// slots whose largest entry lies below its threshold; top_k == 1 (greedy, what top_p == 0 normalises to) skips the
// bisection.  Randomness is counter-based Philox4x32-10 keyed by (seed; row, step) instead of a
// per-row cuRAND state seeded from the wall clock (src/rwkv_sampler.cpp:14-19), so a run is reproducible.
#include <cfloat>

#include "ops.h"

namespace rwkv {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;

__device__ __forceinline__ float sf(float x) {
  const float y = isnan(x) ? 0.0f : x;
  return isinf(y) ? copysignf(FLT_MAX, y) : y;
}

struct BlockRed {
  float f[kSampleWaves];
  unsigned u[kSampleWaves];
};

template <typename Op>
__device__ __forceinline__ float block_reduce_f(float v, Op op, float* buf) {
  v = wave_reduce_dpp(v, op);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) buf[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = buf[0];
#pragma unroll
  for (int i = 1; i < kSampleWaves; ++i) r = op(r, buf[i]);
  return r;
}

__device__ __forceinline__ unsigned block_sum_u(unsigned v, unsigned* buf) {
  v = wave_reduce_dpp(v, [](unsigned x, unsigned y) { return x + y; });
  __syncthreads();
  if ((threadIdx.x & 63) == 0) buf[threadIdx.x >> 6] = v;
  __syncthreads();
  unsigned r = 0;
#pragma unroll
  for (int i = 0; i < kSampleWaves; ++i) r += buf[i];
  return r;
}

// exclusive prefix over threads (thread order), total returned through *total
__device__ __forceinline__ float block_exclusive_scan(float v, float* buf, float* total) {
  float inc = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const float n = __shfl_up(inc, off, 64);
    if ((threadIdx.x & 63) >= off) inc += n;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 63) buf[threadIdx.x >> 6] = inc;
  __syncthreads();
  float base = 0.0f, tot = 0.0f;
#pragma unroll
  for (int i = 0; i < kSampleWaves; ++i) {
    if (i < static_cast<int>(threadIdx.x >> 6)) base += buf[i];
    tot += buf[i];
  }
  *total = tot;
  return base + inc - v;
}

struct Philox {
  uint32_t c[4];
};
__device__ __forceinline__ Philox philox4x32_10(uint64_t seed, uint64_t ctr_lo, uint64_t ctr_hi) {
  uint32_t k0 = static_cast<uint32_t>(seed), k1 = static_cast<uint32_t>(seed >> 32);
  Philox p = {{static_cast<uint32_t>(ctr_lo), static_cast<uint32_t>(ctr_lo >> 32), static_cast<uint32_t>(ctr_hi),
               static_cast<uint32_t>(ctr_hi >> 32)}};
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * p.c[0];
    const uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * p.c[2];
    const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ p.c[1] ^ k0;
    const uint32_t n1 = static_cast<uint32_t>(p1);
    const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ p.c[3] ^ k1;
    const uint32_t n3 = static_cast<uint32_t>(p0);
    p.c[0] = n0; p.c[1] = n1; p.c[2] = n2; p.c[3] = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return p;
}

struct SampleArgs {
  const float* logits;
  float* penalties;  // may be NULL
  float* probs;
  int* out;
  int V;
  float presence, frequency, decay, log2_inv_temp;
  int top_k;
  float top_p;
  uint64_t seed, step;
};

// count and mass of one bisection step through one LDS exchange (the same sums, in the same order, as
// block_sum_u and block_reduce_f one after the other)
__device__ __forceinline__ void block_count_mass(unsigned& c, float& m, BlockRed& red) {
  c = wave_reduce_dpp(c, [](unsigned x, unsigned y) { return x + y; });
  m = wave_reduce_dpp(m, [](float x, float y) { return x + y; });
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    red.u[threadIdx.x >> 6] = c;
    red.f[threadIdx.x >> 6] = m;
  }
  __syncthreads();
  unsigned rc = 0;
  float rm = red.f[0];
#pragma unroll
  for (int i = 0; i < kSampleWaves; ++i) rc += red.u[i];
#pragma unroll
  for (int i = 1; i < kSampleWaves; ++i) rm += red.f[i];
  c = rc;
  m = rm;
}

constexpr int kSampleRegVecs = 16;  // float4 per thread held in registers: rows of up to 65536 entries

// REG: a thread's slice of the row (up to 16 float4) stays in registers from the first load to the draw, so
// the softmax, the ~30 bisection steps and the tie count touch no memory; `probs` is not written.  Larger
// rows keep the slice in `probs` (L2) and re-read it in every pass.  Same arithmetic in the same order.
template <bool REG>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(SampleArgs a) {
  __shared__ BlockRed red;
  __shared__ int s_pick;
  const int b = blockIdx.x;
  const int t = threadIdx.x;
  const int V = a.V;
  const float* logits = a.logits + static_cast<int64_t>(b) * V;
  float* pen = a.penalties ? a.penalties + static_cast<int64_t>(b) * V : nullptr;
  float* probs = a.probs + static_cast<int64_t>(b) * V;
  // contiguous slice per thread, in units of 4 floats
  const int V4 = V / 4;
  const int per = (V4 + kSampleThreads - 1) / kSampleThreads;
  const int i0 = min(t * per, V4);
  const int i1 = min(i0 + per, V4);
  // REG: thread t owns the float4 t, t + 1024, ... (every load of a wavefront is one contiguous KiB); the draw
  // walks the kept entries thread by thread, a fixed permutation of the row, which leaves every entry its probability.
  const int n = REG ? (t < V4 ? min((V4 - t + kSampleThreads - 1) / kSampleThreads, kSampleRegVecs) : 0) : i1 - i0;
  auto fmax_op = [](float x, float y) { return fmaxf(x, y); };
  auto fmin_op = [](float x, float y) { return fminf(x, y); };
  auto fadd_op = [](float x, float y) { return x + y; };

  float4_t vals[REG ? kSampleRegVecs : 1];
  // f(q, i): q = position in the slice, i = float4 index in the row
  auto for_each = [&](auto&& f) {
    if constexpr (REG) {
#pragma unroll
      for (int q = 0; q < kSampleRegVecs; ++q)
        if (q < n) f(q, q * kSampleThreads + t);
    } else {
      for (int i = i0; i < i1; ++i) f(0, i);
    }
  };
  auto get = [&](int q, int i) -> float4_t {
    if constexpr (REG) return vals[q];
    else return reinterpret_cast<const float4_t*>(probs)[i];
  };
  auto put = [&](int q, int i, const float4_t& v) {
    if constexpr (REG) vals[q] = v;
    else reinterpret_cast<float4_t*>(probs)[i] = v;
  };

  // 1. penalised, temperature-scaled logits in base-2 units; row maximum and its lowest index
  if constexpr (REG) {
#pragma unroll
    for (int q = 0; q < kSampleRegVecs; ++q)  // all loads of the slice in flight together
      if (q < n) vals[q] = reinterpret_cast<const float4_t*>(logits)[q * kSampleThreads + t];
  }
  float maxu = -INFINITY;
  int maxi = 0x7fffffff;
  for_each([&](int q, int i) {
    float4_t l;
    if constexpr (REG) l = vals[q];
    else l = reinterpret_cast<const float4_t*>(logits)[i];
    float4_t p = {0.0f, 0.0f, 0.0f, 0.0f};
    if (pen) p = reinterpret_cast<const float4_t*>(pen)[i];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      l[j] = sf((sf(l[j]) - p[j]) * a.log2_inv_temp);
      if (l[j] > maxu) {
        maxu = l[j];
        maxi = i * 4 + j;
      }
    }
    put(q, i, l);
  });
  const float gmax = block_reduce_f(maxu, fmax_op, red.f);
  int pick = -1;

  if (a.top_k == 1) {
    // greedy: lowest index among the maxima (the reference draws uniformly among exact ties)
    unsigned cand = (maxu == gmax) ? static_cast<unsigned>(maxi) : 0x7fffffffu;
    cand = wave_reduce_dpp(cand, [](unsigned x, unsigned y) { return min(x, y); });
    __syncthreads();
    if ((t & 63) == 0) red.u[t >> 6] = cand;
    __syncthreads();
    unsigned best = red.u[0];
#pragma unroll
    for (int i = 1; i < kSampleWaves; ++i) best = min(best, red.u[i]);
    pick = static_cast<int>(best);
  } else {
    // 2.-3. softmax
    float den = 0.0f;
    for_each([&](int q, int i) {
      const float4_t l = get(q, i);
      const float4_t e = {exp2f(l[0] - gmax), exp2f(l[1] - gmax), exp2f(l[2] - gmax), exp2f(l[3] - gmax)};
      den += e[0] + e[1] + e[2] + e[3];
      if constexpr (REG) put(q, i, e);  // registers keep the exponentials for the division below
    });
    den = block_reduce_f(den, fadd_op, red.f);
    float pmax = -INFINITY, pmin = INFINITY;
    for_each([&](int q, int i) {
      float4_t l = get(q, i);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        l[j] = (REG ? l[j] : exp2f(l[j] - gmax)) / den;
        pmax = fmaxf(pmax, l[j]);
        pmin = fminf(pmin, l[j]);
      }
      put(q, i, l);
    });
    // REG: the largest probability among the 256 entries that this wavefront holds in slot q (bit pattern; the same
    // in every lane).  A bisection step whose threshold lies above it has nothing to count there.
    unsigned slot_max[REG ? kSampleRegVecs : 1];
    const bool bisect = a.top_k < V || a.top_p < 1.0f;  // (else the loop below does not run: no threshold to find)
    if constexpr (REG) {
#pragma unroll
      for (int q = 0; q < kSampleRegVecs; ++q) slot_max[q] = 0xffffffffu;
    }
    if (REG && bisect) {
#pragma unroll
      for (int q = 0; q < kSampleRegVecs; ++q) {
        float mx = 0.0f;
        if (q < n) mx = fmaxf(fmaxf(vals[q][0], vals[q][1]), fmaxf(vals[q][2], vals[q][3]));
        mx = wave_reduce_dpp(mx, fmax_op);
        slot_max[q] = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, mx)));
      }
    }
    pmax = block_reduce_f(pmax, fmax_op, red.f);
    pmin = block_reduce_f(pmin, fmin_op, red.f);

    // 4. threshold by bisection on the bit pattern
    unsigned left = __float_as_uint(pmin), right = __float_as_uint(pmax) + 1u;
    unsigned cnt = static_cast<unsigned>(V);
    float mass = 1.0f;
    while ((cnt > static_cast<unsigned>(a.top_k) || mass > a.top_p) && left < right - 1u) {
      const unsigned mid = left + (right - left) / 2u;
      const float thr = __uint_as_float(mid);
      unsigned c = 0;
      float m = 0.0f;
      if constexpr (REG) {
        // (probabilities are not negative: their order is the order of their bit patterns, which the bisection
        // itself relies on; the comparison of two wavefront-wide values is a scalar one)
        const unsigned mid_u = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(mid)));
#pragma unroll
        for (int q = 0; q < kSampleRegVecs; ++q) {
          if (slot_max[q] >= mid_u) {
            if (q < n) {
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (vals[q][j] >= thr) {
                  ++c;
                  m += vals[q][j];
                }
            }
          }
        }
      } else {
        for_each([&](int q, int i) {
          const float4_t l = get(q, i);
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (l[j] >= thr) {
              ++c;
              m += l[j];
            }
        });
      }
      block_count_mass(c, m, red);
      if (c < static_cast<unsigned>(a.top_k) && m < a.top_p) {
        right = mid;
      } else {
        left = mid;
        cnt = c;
        mass = m;
      }
    }
    const float thr = __uint_as_float(left);

    // 5. tie compensation
    unsigned eqk = 0, gtk = 0;
    float gtp = 0.0f;
    for_each([&](int q, int i) {
      const float4_t l = get(q, i);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (l[j] == thr) ++eqk;
        if (l[j] > thr) {
          ++gtk;
          gtp += l[j];
        }
      }
    });
    const unsigned n_eq = block_sum_u(eqk, red.u);
    const unsigned n_gt = block_sum_u(gtk, red.u);
    const float p_gt = block_reduce_f(gtp, fadd_op, red.f);
    float comp = 1.0f;
    if (n_eq > 0) {
      comp = fminf(sf((a.top_p - p_gt) / (thr * n_eq)), comp);
      comp = fminf(sf(static_cast<float>(a.top_k - static_cast<int>(n_gt)) / n_eq), comp);
      comp = fmaxf(comp, 0.0f);
    }

    // 6. inverse-CDF draw over the kept set, thread by thread
    const float mine = gtp + (thr * eqk) * comp;
    float total;
    const float before = block_exclusive_scan(mine, red.f, &total);
    const Philox rnd = philox4x32_10(a.seed, static_cast<uint64_t>(b), a.step);
    // uniform in (0,1]: never selects a zero-mass prefix
    const float u = (static_cast<float>(rnd.c[0] >> 8) + 1.0f) * (1.0f / 16777216.0f);
    const float target = u * total;
    if (t == 0) s_pick = -1;
    __syncthreads();
    if (mine > 0.0f && target > before && target <= before + mine) {
      float cum = before;
      int found = -1, last = -1;
      for_each([&](int q, int i) {
        const float4_t l = get(q, i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float w = (l[j] < thr) ? 0.0f : (l[j] == thr ? l[j] * comp : l[j]);
          if (w > 0.0f && found < 0) {
            cum += w;
            last = i * 4 + j;
            if (cum >= target) found = last;
          }
        }
      });
      if (found < 0) found = last;  // rounding inside the slice: its last kept entry
      atomicMax(&s_pick, found);
    }
    __syncthreads();
    const bool fallback = s_pick < 0;  // rounding between slices left the target past every interval
    __syncthreads();
    if (fallback && mine > 0.0f) {
      int last = -1;
      for_each([&](int q, int i) {
        const float4_t l = get(q, i);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (l[j] > thr || (l[j] == thr && comp > 0.0f)) last = i * 4 + j;
      });
      atomicMax(&s_pick, last);
    }
    __syncthreads();
    pick = s_pick < 0 ? 0 : s_pick;
  }

  if (t == 0) a.out[b] = pick;
  // 7. penalty update (sampling.cu:461-470)
  if (pen) {
    for_each([&](int, int i) {
      float4_t p = reinterpret_cast<float4_t*>(pen)[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float add = (pick != i * 4 + j) ? 0.0f : (p[j] == 0.0f ? a.presence : a.frequency);
        p[j] = fmaf(p[j], a.decay, add);
      }
      reinterpret_cast<float4_t*>(pen)[i] = p;
    });
  }
}

// One 1024-thread block per row; 16-byte loads, eight in flight per thread (the row is 256 KiB at V = 65536 and
// the kernel is pure load latency).  Lowest index among equal maxima.
constexpr int kArgmaxThreads = 1024;

// next / history (may be null): the picked id also becomes the row's next input token and an entry of the caller's
// list of generated tokens - what a greedy decode loop would otherwise launch a second kernel for.
__global__ __launch_bounds__(kArgmaxThreads) void argmax_kernel(int V, const float* __restrict__ logits, int* __restrict__ out,
                                                               int64_t* __restrict__ next, int* __restrict__ history) {
  __shared__ float bv[kArgmaxThreads / 64];
  __shared__ int bi[kArgmaxThreads / 64];
  const float* row = logits + static_cast<int64_t>(blockIdx.x) * V;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  auto take = [&](float v, int i) {
    if (v > best || (v == best && i < idx)) {
      best = v;
      idx = i;
    }
  };
  const bool vec_ok = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  const int V4 = vec_ok ? V / 4 : 0;
  constexpr int kBatch = 8;
  for (int base = 0; base < V4; base += kArgmaxThreads * kBatch) {
    float4_t q[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = base + u * kArgmaxThreads + threadIdx.x;
      q[u] = float4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (i < V4) q[u] = reinterpret_cast<const float4_t*>(row)[i];
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int i = (base + u * kArgmaxThreads + threadIdx.x) * 4;
      if (i < V4 * 4) {
        take(q[u].x, i);
        take(q[u].y, i + 1);
        take(q[u].z, i + 2);
        take(q[u].w, i + 3);
      }
    }
  }
  for (int i = V4 * 4 + threadIdx.x; i < V; i += kArgmaxThreads) take(row[i], i);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(idx, off, 64);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    bv[threadIdx.x >> 6] = best;
    bi[threadIdx.x >> 6] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < kArgmaxThreads / 64; ++i)
      if (bv[i] > best || (bv[i] == best && bi[i] < idx)) {
        best = bv[i];
        idx = bi[i];
      }
    const int pick = idx == 0x7fffffff ? 0 : idx;
    out[blockIdx.x] = pick;
    if (next) next[blockIdx.x] = pick;
    if (history) history[blockIdx.x] = pick;
  }
}

int argmax_launch(hipStream_t st, int B, int V, const float* logits, int* out, int64_t* next, int* history) {
  hipLaunchKernelGGL(argmax_kernel, dim3(B), dim3(kArgmaxThreads), 0, st, V, logits, out, next, history);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_sample(rwkv_stream_t s, int B, int V, const void* logits, void* penalties, void* probs, void* out,
                    double presence, double frequency, double decay, double temperature, int top_k, double top_p,
                    uint64_t seed, uint64_t step) {
  // same argument checks as the reference (src/utils/sampling.cu:492-512)
  RWKV_REQUIRE(V > 0 && V <= 1048576 && V % 4 == 0,
               "Vocabulary size must be multiple of 4, and no larger than 1048576, got %d", V);
  RWKV_REQUIRE(B > 0, "B must be positive, got %d", B);
  RWKV_REQUIRE(temperature >= 0.001 && temperature <= 1000.0, "Temperature outside range, got %f", temperature);
  RWKV_REQUIRE(logits && probs && out, "sample: NULL tensor");
  if (top_k <= 0 || top_k > V) top_k = V;
  if (top_p < 0 || top_p > 1) top_p = 1;
  if (top_p == 0) {
    top_k = 1;
    top_p = 1;
  }
  SampleArgs a;
  a.logits = static_cast<const float*>(logits);
  a.penalties = static_cast<float*>(penalties);
  a.probs = static_cast<float*>(probs);
  a.out = static_cast<int*>(out);
  a.V = V;
  a.presence = static_cast<float>(presence);
  a.frequency = static_cast<float>(frequency);
  a.decay = static_cast<float>(decay);
  a.log2_inv_temp = static_cast<float>(1.44269504088896340736 / temperature);
  a.top_k = top_k;
  a.top_p = static_cast<float>(top_p);
  a.seed = seed;
  a.step = step;
  if (V / 4 <= kSampleRegVecs * kSampleThreads) {
    hipLaunchKernelGGL(sample_kernel<true>, dim3(B), dim3(kSampleThreads), 0, as_stream(s), a);
  } else {
    hipLaunchKernelGGL(sample_kernel<false>, dim3(B), dim3(kSampleThreads), 0, as_stream(s), a);
  }
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int rwkv_hip_argmax(rwkv_stream_t s, int B, int V, const void* logits, void* out) {
  RWKV_REQUIRE(B > 0 && V > 0 && logits && out, "argmax: bad arguments");
  return argmax_launch(as_stream(s), B, V, static_cast<const float*>(logits), static_cast<int*>(out));
}

}  // extern "C"
