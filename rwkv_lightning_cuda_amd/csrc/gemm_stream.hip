// Weight-streaming MFMA GEMM Y[M,N] = X[M,K] . W[N,K]^T over weights stored in an MFMA-native packed order.
// This is the M >= 16 path of the model: batched decode (M = batch) and prefill chunks (M = batch * 128).
//
// Reference: the cuBLAS / cuBLASLt calls behind rwkv7_v3a_linear_f16_orig_launch and
// rwkv7_v3a_linear_f16_orig_lt_cfg_launch (cuda/rwkv7_v3a_ops.cu:2235-2368): fp16 in, fp32 accumulate, fp16
// (or fp32) out.  The arithmetic there lives in a closed library; the contract is the textbook GEMM.
//
// Packed order.  v_mfma_f32_32x32x16_f16 takes, from lane l = j + 32h, 8 fp16 values of row j of each
// operand for 8 of the 16 k of the step; any assignment of k to (h, step) is valid as long as both operands
// use the same one.  A packed matrix is cut into tiles of 32 rows x G k (G = 32 for fp16 and int8 codes, 64
// for int4 codes); inside a tile lane (j, h) owns the KR = G/2 consecutive k [h*KR, h*KR + KR) of row j, and
// the tile is stored as 64 lanes x 16 bytes (x 2 pieces for fp16), tiles of one 32-row band consecutive
// along k.  A wavefront therefore streams one band with 1 KiB fully coalesced loads and feeds the pieces
// to the matrix core after an exact in-register expansion of the codes, without any transpose or LDS
// traffic for the weights; every weight byte leaves HBM once per 32*MT rows of X.
//
// Work split.  A block covers 32*MT rows x 128 output columns x one K slice with one or two groups of four
// wavefronts: each wavefront streams one band, the groups take alternate chunks of KC = 128 k and meet in LDS at
// the end.  The X rows of a chunk are staged in LDS and shared by the four wavefronts of the group.  Chunks
// are software-pipelined: weight pieces are requested three chunks ahead into a ring of register sets, X two
// chunks ahead, the X fragments of the next MFMA step are read from LDS while the current one runs; one barrier
// per chunk.  With more than one K split each block writes an fp32 partial tile and a second small kernel
// sums the partials in split order (a fixed order: results do not depend on scheduling) and applies scale and
// epilogue.
#include <algorithm>
#include <cstdlib>

#include "ops.h"

namespace rwkv {

typedef float float16_t __attribute__((ext_vector_type(16)));

template <int FMT>
struct PackTraits;
template <>
struct PackTraits<RWKV_FMT_F16> {
  static constexpr int KR = 16, PIECES = 2;
};
template <>
struct PackTraits<RWKV_FMT_W8> {
  static constexpr int KR = 16, PIECES = 1;
};
template <>
struct PackTraits<RWKV_FMT_W4> {
  static constexpr int KR = 32, PIECES = 1;
};

bool linear_packed_supported(int fmt, int M, int N, int K) {
  if (fmt != RWKV_FMT_F16 && fmt != RWKV_FMT_W8 && fmt != RWKV_FMT_W4) return false;
  return M >= 1 && N >= 32 && N % 32 == 0 && K >= 256 && K % 256 == 0;
}

// ---- packing: a permutation of the 16-byte pieces of the row-major codes ---------------------------------------------
__global__ __launch_bounds__(256) void pack_weights_kernel(int fmt, int N, int K, const uint4_t* __restrict__ src,
                                                           uint4_t* __restrict__ dst, int64_t n_pieces) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (p >= n_pieces) return;
  const int G = fmt == RWKV_FMT_W4 ? 64 : 32;
  const int KR = G / 2;
  const int pieces = fmt == RWKV_FMT_F16 ? 2 : 1;
  const int lane = static_cast<int>(p & 63);
  int64_t q = p >> 6;
  const int i = static_cast<int>(q % pieces);
  q /= pieces;
  const int KG = K / G;
  const int kg = static_cast<int>(q % KG);
  const int nt = static_cast<int>(q / KG);
  const int row = nt * 32 + (lane & 31);
  const int k = kg * G + (lane >> 5) * KR + i * 8;
  // elements per 16-byte piece: 8 (fp16), 16 (int8), 32 (int4)
  const int per = fmt == RWKV_FMT_F16 ? 8 : (fmt == RWKV_FMT_W8 ? 16 : 32);
  dst[p] = src[(static_cast<int64_t>(row) * K + k) / per];
}

int pack_weights_launch(hipStream_t st, int fmt, int N, int K, const void* w, void* packed) {
  RWKV_REQUIRE(linear_packed_supported(fmt, 16, N, K), "pack_weights: unsupported shape N=%d K=%d fmt=%d", N, K, fmt);
  RWKV_REQUIRE(w && packed && w != packed, "pack_weights: bad pointers");
  const int per = fmt == RWKV_FMT_F16 ? 8 : (fmt == RWKV_FMT_W8 ? 16 : 32);
  const int64_t n_pieces = static_cast<int64_t>(N) * K / per;
  hipLaunchKernelGGL(pack_weights_kernel, dim3(static_cast<unsigned>((n_pieces + 255) / 256)), dim3(256), 0, st, fmt,
                     N, K, static_cast<const uint4_t*>(w), static_cast<uint4_t*>(packed), n_pieces);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

// ---- the GEMM ---------------------------------------------------------------------------------------------------------

struct StreamProblem {
  const half_t* x;
  const uint4_t* wp;
  const half_t* scale;
  const uint8_t* zp;
  void* y;
  float* partial;  // [splits][M][N] fp32, only with splits > 1
  int N;
  int fmt;
};

// Up to kMaxProblems products that share M, K and the split (each with its own weights, format, x and y) in one
// launch: grid.y runs over the column blocks of all problems, block_end[] are the prefix sums.
struct StreamArgs {
  StreamProblem p[kMaxProblems];
  int block_end[kMaxProblems];
  int n_problems;
  int M, K;
  int splits, k_per_split;
  int row_tiles, col_blocks;
  int epilogue, out_f32;
  RowCopy copy;  // rides on the launch: its first blocks move these rows (they are no operand of the product)
};

// shared out between the first blocks of the launch, so that no single block carries it on its critical path
__device__ __forceinline__ void ride_along_copy(const RowCopy& cp) {
  constexpr unsigned kCopyBlocks = 8;
  const unsigned nb = gridDim.x < kCopyBlocks ? gridDim.x : kCopyBlocks;
  if (blockIdx.x < nb && blockIdx.y == 0 && blockIdx.z == 0 && cp.n > 0) {
    for (int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8; i < cp.n; i += nb * blockDim.x * 8)
      *reinterpret_cast<uint4_t*>(cp.dst + i) = *reinterpret_cast<const uint4_t*>(cp.src + i);
  }
}

__device__ __forceinline__ half8_t make_half8(half2_t a, half2_t b, half2_t c, half2_t d) {
  half8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
  r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
  return r;
}

// 8 int8 codes (two dwords) -> 8 fp16, exact: byte^0x80 under exponent 0x64 is 1024 + (code + 128).
__device__ __forceinline__ half8_t expand_w8(uint32_t d0, uint32_t d1) {
  const half2_t bias = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};
  d0 ^= 0x80808080u;
  d1 ^= 0x80808080u;
  return make_half8(as_half2(__builtin_amdgcn_perm(0x64646464u, d0, 0x04010400u)) - bias,
                    as_half2(__builtin_amdgcn_perm(0x64646464u, d0, 0x04030402u)) - bias,
                    as_half2(__builtin_amdgcn_perm(0x64646464u, d1, 0x04010400u)) - bias,
                    as_half2(__builtin_amdgcn_perm(0x64646464u, d1, 0x04030402u)) - bias);
}

// 8 int4 codes (one dword, element 2i in the low nibble of byte i) minus the zero point -> 8 fp16, exact.
__device__ __forceinline__ half8_t expand_w4(uint32_t d, half2_t bias) {
  const uint32_t even = d & 0x0f0f0f0fu;
  const uint32_t odd = (d >> 4) & 0x0f0f0f0fu;
  return make_half8(as_half2(__builtin_amdgcn_perm(odd, even, 0x0c040c00u) | 0x64006400u) - bias,
                    as_half2(__builtin_amdgcn_perm(odd, even, 0x0c050c01u) | 0x64006400u) - bias,
                    as_half2(__builtin_amdgcn_perm(odd, even, 0x0c060c02u) | 0x64006400u) - bias,
                    as_half2(__builtin_amdgcn_perm(odd, even, 0x0c070c03u) | 0x64006400u) - bias);
}

template <int FMT, int MT, int KC, int WG = 4>
struct Tile {
  using P = PackTraits<FMT>;
  static constexpr int BM = 32 * MT;
  static constexpr int G = 2 * P::KR;
  static constexpr int GROUPS = KC / G;
  static constexpr int NW = GROUPS * P::PIECES;     // weight pieces per lane per chunk
  static constexpr int STEPS = P::KR / 8;
  static constexpr int XSTRIDE = KC + 8;            // fp16 per staged row: 16-byte pad keeps b128 reads conflict-free
  static constexpr int GT = 64 * WG;                // threads of a wavefront group
  static constexpr int XV = BM * (KC / 8) / GT;     // 16-byte vectors of X per thread per chunk
  static constexpr int QG = KC / 128;               // int4 scale groups per chunk
  static constexpr int NACC = MT == 1 ? 2 : 1;      // independent accumulation chains per row tile
  static constexpr int DEPTH = (NW * 4 <= 16) ? 4 : (NW * 4 <= 32 ? 3 : 2);  // weight register sets in the ring
  static constexpr int kTileHalfs = BM * XSTRIDE;   // one staged X tile
  static_assert(KC % 128 == 0 && XV >= 1, "chunk must hold whole int4 groups and at least one vector per thread");
};

__device__ __forceinline__ float finish_value(float v, int epilogue) {
  v = round_h(v);
  if (epilogue == RWKV_EPI_RELU_SQUARE) {
    v = fmaxf(v, 0.0f);
    v = round_h(v * v);
  }
  return v;
}

// One chunk's slice of X held by a thread between request and its store to LDS.
template <int FMT, int MT, int KC, int WG>
struct XRegs {
  using T = Tile<FMT, MT, KC, WG>;
  uint4_t xv[T::XV];

  // vector i of the thread's slice
  __device__ __forceinline__ void request_one(int i, const StreamArgs& g, const StreamProblem& pr, int tid, int m0, int kc) {
    const int idx = tid + i * T::GT;
    const int r = idx / (KC / 8);
    const int c = (idx % (KC / 8)) * 8;
    // rows past M repeat the last row (their sums are never stored): a load under a per-lane branch, or merged
    // with a default value, makes the compiler drain every load in flight at the head of the chunk loop
    const int row = m0 + r < g.M ? m0 + r : g.M - 1;
    xv[i] = *reinterpret_cast<const uint4_t*>(pr.x + static_cast<int64_t>(row) * g.K + kc + c);
  }
  __device__ __forceinline__ void store_one(int i, int tid, half_t* xs) const {
    const int idx = tid + i * T::GT;
    const int r = idx / (KC / 8);
    const int c = (idx % (KC / 8)) * 8;
    *reinterpret_cast<uint4_t*>(xs + r * T::XSTRIDE + c) = xv[i];
  }

  __device__ __forceinline__ void request(const StreamArgs& g, const StreamProblem& pr, int tid, int m0, int kc) {
#pragma unroll
    for (int i = 0; i < T::XV; ++i) request_one(i, g, pr, tid, m0, kc);
  }

  __device__ __forceinline__ void store_x(int tid, half_t* xs) const {
#pragma unroll
    for (int i = 0; i < T::XV; ++i) store_one(i, tid, xs);
  }
};

// One chunk's weight pieces (and int4 group scales) held by a lane between request and use.
template <int FMT, int MT, int KC>
struct WRegs {
  using T = Tile<FMT, MT, KC>;
  uint4_t w[T::NW];
  // int4 group scale and zero point as loaded: converted at their use in multiply().  Converted beside the loads,
  // they would make every request wait for all the weights in flight.
  half_t sc[T::QG];
  uint32_t zb[T::QG];

  // piece i of the chunk at kc (fp16 and int8 codes: no group scales)
  __device__ __forceinline__ void request_piece(int i, int kc, const uint4_t* wband) {
    using P = typename T::P;
    w[i] = wband[static_cast<int64_t>(kc / T::G) * (P::PIECES * 64) + i * 64];
  }

  __device__ __forceinline__ void request(const StreamArgs& g, const StreamProblem& pr, int kc, const uint4_t* wband,
                                          int n) {
    using P = typename T::P;
    const uint4_t* wp = wband + static_cast<int64_t>(kc / T::G) * (P::PIECES * 64);
#pragma unroll
    for (int i = 0; i < T::NW; ++i) w[i] = wp[i * 64];
    if constexpr (FMT == RWKV_FMT_W4) {
      const int64_t q0 = static_cast<int64_t>(n) * (g.K >> 7) + (kc >> 7);
#pragma unroll
      for (int q = 0; q < T::QG; ++q) {
        sc[q] = pr.scale[q0 + q];
        zb[q] = pr.zp[q0 + q];
      }
    }
  }

  // The X fragments of MFMA step ks+1 are read from LDS while step ks runs (the compiler on its own issues each
  // read right before its use, which leaves the matrix core idle for the LDS latency on every step);
  // __builtin_amdgcn_sched_barrier(0) keeps the reads where they are written.
  __device__ __forceinline__ void multiply(const half_t* xs, int j, int h, float16_t (&acc)[MT][T::NACC],
                                           float16_t (&part)[MT][T::NACC]) const {
    using P = typename T::P;
    constexpr int NK = T::GROUPS * T::STEPS;
    float scf[T::QG], zbf[T::QG];
    if constexpr (FMT == RWKV_FMT_W4) {
#pragma unroll
      for (int q = 0; q < T::QG; ++q) {
        uint32_t sr = __builtin_bit_cast(unsigned short, sc[q]), zr = zb[q];
        asm volatile("" : "+v"(sr), "+v"(zr));  // the conversions stay here, below the requests of this chunk
        scf[q] = h2f(__builtin_bit_cast(half_t, static_cast<unsigned short>(sr)));
        zbf[q] = 1024.0f + static_cast<float>(zr);
      }
    }
    const half_t* xlane = xs + j * T::XSTRIDE + h * P::KR;
    half8_t a[2][MT];
    auto load_a = [&](int ks, half8_t (&dst)[MT]) {
      const half_t* xa = xlane + (ks / T::STEPS) * T::G + 8 * (ks % T::STEPS);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) dst[mt] = *reinterpret_cast<const half8_t*>(xa + mt * 32 * T::XSTRIDE);
    };
    load_a(0, a[0]);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      const int gi = ks / T::STEPS;
      const int s = ks % T::STEPS;
      if (ks + 1 < NK) load_a(ks + 1, a[(ks + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      half8_t b;
      if constexpr (FMT == RWKV_FMT_F16) {
        const uint4_t piece = w[gi * 2 + s];
        b = __builtin_bit_cast(half8_t, piece);
      } else if constexpr (FMT == RWKV_FMT_W8) {
        const uint4_t piece = w[gi];
        b = s == 0 ? expand_w8(piece[0], piece[1]) : expand_w8(piece[2], piece[3]);
      } else {
        const uint4_t piece = w[gi];
        const half_t zf = static_cast<half_t>(zbf[(gi * T::G) >> 7]);
        const half2_t bias = {zf, zf};
        b = expand_w4(piece[s], bias);
      }
      constexpr int kChainMask = T::NACC - 1;
      const int chain = ks & kChainMask;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if constexpr (FMT == RWKV_FMT_W4) {
          part[mt][chain] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks & 1][mt], b, part[mt][chain], 0, 0, 0);
        } else {
          acc[mt][chain] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks & 1][mt], b, acc[mt][chain], 0, 0, 0);
        }
      }
      if constexpr (FMT == RWKV_FMT_W4) {
        if (s == T::STEPS - 1 && ((gi + 1) * T::G) % 128 == 0) {  // end of a 128-group: fold with its scale
          const float s128 = scf[(gi * T::G) >> 7];
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int c = 0; c < T::NACC; ++c)
#pragma unroll
              for (int v = 0; v < 16; ++v) {
                acc[mt][c][v] = fmaf(part[mt][c][v], s128, acc[mt][c][v]);
                part[mt][c][v] = 0.0f;
              }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// One block of one problem: 32 * WG columns x the block's K slice.  The block has KG groups of WG wavefronts (one
// 32-column band of the weights per wavefront); group kg takes chunks kg, kg + KG, ... of the slice with its own
// pair of X tiles in LDS, and the groups' sums meet in LDS at the end (in group order), so that a CU holds two
// wavefronts per SIMD - one's code expansion overlaps the other's matrix-core time - without more fp32 partial
// tiles in HBM.
//
// Per group and chunk c: the X slice of chunk c+2 is requested into registers, the weight pieces of chunk
// c+D-1 into a ring of D register sets, the matrix core runs chunk c out of LDS tile c&1, then the X slice of
// chunk c+1 (requested one iteration earlier) is stored to the other tile; one barrier per chunk.  Every load
// of the loop is issued unconditionally - past the end of the slice it re-reads the current chunk, which is in
// cache - because a load under a branch makes the compiler's s_waitcnt accounting assume the shorter path
// and wait for everything in flight.  Within an iteration X is requested before the weights, so that waiting
// for X does not wait for the younger weight loads.
template <int FMT, int MT, int KC, int KG, int WG>
__device__ __forceinline__ void stream_block(const StreamArgs& g, const StreamProblem& pr, int row_tile, int col_block,
                                             int split, half_t* xs_all) {
  using T = Tile<FMT, MT, KC, WG>;
  using P = typename T::P;
  constexpr int BM = T::BM;
  constexpr int GT = T::GT;

  const int tid = threadIdx.x % GT;  // thread within its k-group
  const int kg = threadIdx.x / GT;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int m0 = row_tile * BM;
  const int band_here = col_block * WG + wave;  // 32-row band of W = 32 output columns
  const bool active = band_here * 32 < pr.N;
  const int band = active ? band_here : pr.N / 32 - 1;  // a wavefront past the last band repeats it and stores nothing
  const int n = band * 32 + j;
  constexpr int KSTRIDE = KC * KG;  // between consecutive chunks of one group
  const int kbeg = split * g.k_per_split + kg * KC;
  const int nchunks = g.k_per_split / KSTRIDE;
  half_t* xs = xs_all + kg * 2 * T::kTileHalfs;

  float16_t acc[MT][T::NACC], part[MT][T::NACC];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int c = 0; c < T::NACC; ++c)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        acc[mt][c][v] = 0.0f;
        part[mt][c][v] = 0.0f;
      }

  // this lane's first piece of the band; consecutive pieces are 64 uint4 apart
  const uint4_t* wband = pr.wp + (static_cast<int64_t>(band) * (g.K / T::G)) * (P::PIECES * 64) + lane;
  // the column's int8 scale now: read in the epilogue it costs every block a trip to memory (1.2 us per launch)
  half_t scale_h = static_cast<half_t>(1.0f);
  if constexpr (FMT == RWKV_FMT_W8) scale_h = pr.scale[n];

  constexpr int D = T::DEPTH;
  WRegs<FMT, MT, KC> wr[D];
  XRegs<FMT, MT, KC, WG> xr[2];
  const int last = nchunks - 1;
  xr[0].request(g, pr, tid, m0, kbeg);
  xr[1].request(g, pr, tid, m0, kbeg + min(1, last) * KSTRIDE);
#pragma unroll
  for (int i = 0; i < D - 1; ++i) wr[i].request(g, pr, kbeg + min(i, last) * KSTRIDE, wband, n);
  xr[0].store_x(tid, xs);
  __syncthreads();
  constexpr int U = (D % 2 == 0) ? D : 2 * D;  // unroll: register sets and LDS tiles are indexed statically
  // Whole rounds of U chunks run as one basic block: with an exit between the chunks the compiler waits for every
  // load in flight at the head of each round (the weight ring then drains once per round).  The chunks left over
  // (K slices that are not a multiple of U chunks) take the same steps with the exits.
  const int whole = nchunks - nchunks % U;
  int c0 = 0;
  for (; c0 < whole; c0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u;
      xr[u & 1].request(g, pr, tid, m0, kbeg + (c + 2 <= last ? c + 2 : c) * KSTRIDE);
      wr[(u + D - 1) % D].request(g, pr, kbeg + (c + D - 1 <= last ? c + D - 1 : c) * KSTRIDE, wband, n);
      wr[u % D].multiply(xs + (u & 1) * T::kTileHalfs, j, h, acc, part);
      xr[(u + 1) & 1].store_x(tid, xs + ((u + 1) & 1) * T::kTileHalfs);
      __syncthreads();
    }
  }
  if (c0 < nchunks) {
#pragma unroll
    for (int u = 0; u < U - 1; ++u) {
      const int c = c0 + u;
      if (c >= nchunks) break;
      xr[u & 1].request(g, pr, tid, m0, kbeg + (c + 2 <= last ? c + 2 : c) * KSTRIDE);
      wr[(u + D - 1) % D].request(g, pr, kbeg + (c + D - 1 <= last ? c + D - 1 : c) * KSTRIDE, wband, n);
      wr[u % D].multiply(xs + (u & 1) * T::kTileHalfs, j, h, acc, part);
      xr[(u + 1) & 1].store_x(tid, xs + ((u + 1) & 1) * T::kTileHalfs);
      __syncthreads();
    }
  }

  if constexpr (T::NACC == 2) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mt][0][v] += acc[mt][1][v];
  }
  // The X tiles are free after the last barrier.  The other groups hand their sums to group 0 through them; group 0
  // then lays the finished 32*MT x 32*WG tile out in LDS (rows padded by 8 floats) and all threads write it to
  // memory in 16/32-byte pieces along the rows - the accumulator layout itself would give 2-byte stores 64 bytes
  // apart.
  constexpr int kCols = 32 * WG;         // columns of the block
  constexpr int kStageLd = kCols + 8;
  constexpr int kRedFloats = (KG - 1) * MT * 16 * GT;
  float* stage = reinterpret_cast<float*>(xs_all) + kRedFloats;
  static_assert(kRedFloats * 4 + BM * kStageLd * 4 <= KG * 2 * T::kTileHalfs * 2, "epilogue tile exceeds the LDS tiles");
  if constexpr (KG > 1) {
    float* red = reinterpret_cast<float*>(xs_all);
    if (kg > 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) red[((kg - 1) * MT * 16 + mt * 16 + v) * GT + tid] = acc[mt][0][v];
    }
    __syncthreads();
  }
  const bool partial_out = g.splits > 1;
  if (kg == 0) {
    const float scl = partial_out ? 1.0f : h2f(scale_h);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float sum = acc[mt][0][v];
#pragma unroll
        for (int q = 1; q < KG; ++q) sum += reinterpret_cast<const float*>(xs_all)[((q - 1) * MT * 16 + mt * 16 + v) * GT + tid];
        const int row = mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        stage[row * kStageLd + wave * 32 + j] = partial_out ? sum : finish_value(mul_f32(sum, scl), g.epilogue);
      }
  }
  __syncthreads();
  float* part_out = partial_out ? pr.partial + static_cast<int64_t>(split) * g.M * pr.N : nullptr;
  const int col0 = col_block * kCols;
  constexpr int kPieces = kCols / 8;  // 8-column pieces per row
  for (int idx = threadIdx.x; idx < BM * kPieces; idx += GT * KG) {
    const int row = idx / kPieces;
    const int piece = idx % kPieces;
    const int col = col0 + piece * 8;
    if (m0 + row >= g.M || col >= pr.N) continue;
    const float4_t lo = *reinterpret_cast<const float4_t*>(stage + row * kStageLd + piece * 8);
    const float4_t hi = *reinterpret_cast<const float4_t*>(stage + row * kStageLd + piece * 8 + 4);
    const int64_t o = static_cast<int64_t>(m0 + row) * pr.N + col;
    if (partial_out || g.out_f32) {
      float* dst = partial_out ? part_out + o : static_cast<float*>(pr.y) + o;
      *reinterpret_cast<float4_t*>(dst) = lo;
      *reinterpret_cast<float4_t*>(dst + 4) = hi;
    } else {
      half8_t hv;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        hv[e] = f2h(lo[e]);
        hv[4 + e] = f2h(hi[e]);
      }
      *reinterpret_cast<half8_t*>(static_cast<half_t*>(pr.y) + o) = hv;
    }
  }
}

// grid = row tiles x roundup(column blocks over all problems x splits, 8), one-dimensional; block = 64 * WG * KG.
// Workgroups go to the eight XCDs round-robin by linear id, each XCD with its own L2: the id is decoded so that
// the row tiles of one (column block, split) pair - which stream the same weights - land on the same XCD.
template <int MT, int KC, int KG, int WG>
__global__ __launch_bounds__(64 * WG * KG) void gemm_stream_kernel(StreamArgs g) {
  __shared__ __align__(16) half_t xs[KG * 2 * 32 * MT * (KC + 8)];
  ride_along_copy(g.copy);
  const int id = blockIdx.x;
  const int row_tile = (id >> 3) % g.row_tiles;
  const int pair = (id / (8 * g.row_tiles)) * 8 + (id & 7);
  if (pair >= g.col_blocks * g.splits) return;
  const int col_all = pair % g.col_blocks;
  const int split = pair / g.col_blocks;
  int pi = 0;
  while (pi + 1 < g.n_problems && col_all >= g.block_end[pi]) ++pi;
  const int col_block = col_all - (pi > 0 ? g.block_end[pi - 1] : 0);
  const StreamProblem& pr = g.p[pi];
  switch (pr.fmt) {
    case RWKV_FMT_W8: stream_block<RWKV_FMT_W8, MT, KC, KG, WG>(g, pr, row_tile, col_block, split, xs); break;
    case RWKV_FMT_W4: stream_block<RWKV_FMT_W4, MT, KC, KG, WG>(g, pr, row_tile, col_block, split, xs); break;
    default: stream_block<RWKV_FMT_F16, MT, KC, KG, WG>(g, pr, row_tile, col_block, split, xs); break;
  }
}

// ---- many rows: 128 rows x 256 columns per block, two bands per wavefront -------------------------------------------
// From a few hundred rows on the product is bound by the matrix core and by LDS, not by the weights: with one band
// per wavefront every MFMA needs its own 1 KiB X fragment from LDS, and LDS delivers 128 bytes per clock against
// 32 clocks per MFMA and SIMD - four wavefronts saturate both at once.  Here a wavefront keeps two 32-column bands
// (wave w: bands w and w + 4 of the block), so each X fragment feeds two MFMAs and a block reads X from L2 half as
// often.  One group of four wavefronts, one wavefront per SIMD (128 accumulator registers per lane); int8 and
// fp16 weights (the int4 path would double the accumulators once more and stays on the narrower tile).
//
// ROLL (int8 weights only): the variant that fits two wavefronts per SIMD (at most 256 registers).  Alone on its
// SIMD a wavefront overlaps nothing - measured per 128-k chunk: 1.18 us of MFMAs, and on top of them, one after the
// other, 0.2 us for the weight requests, 0.2 for the X requests and stores, 0.18 for the code expansion, 0.1 for
// the LDS reads - so a second wavefront, whose MFMAs fill those gaps, is worth more than deep prefetch.  The
// registers come from the weights: one set per band instead of a ring of sets, each piece requested again for the
// next chunk right after its last use (six MFMA steps ahead), and from X: one set, requested during the first
// half of a chunk's steps and stored during the second.
template <int FMT, bool ROLL, int MT>
__device__ __forceinline__ void stream_block_wide(const StreamArgs& g, const StreamProblem& pr, int row_tile, int col_block,
                                                  int split, half_t* xs) {
  static_assert(!ROLL || FMT == RWKV_FMT_W8, "the rolling weight set is laid out for int8 pieces (two MFMA steps each)");
  constexpr int KC = 128, NB = 2;
  using T = Tile<FMT, MT, KC, 4>;
  using P = typename T::P;
  constexpr int BM = T::BM;
  static_assert(FMT != RWKV_FMT_W4, "the wide tile takes int8 and fp16 weights");

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int j = lane & 31;
  const int h = lane >> 5;
  const int m0 = row_tile * BM;
  const int kbeg = split * g.k_per_split;
  const int nchunks = g.k_per_split / KC;

  bool active[NB];
  int n[NB];
  const uint4_t* wband[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int band_here = col_block * (4 * NB) + nb * 4 + wave;
    active[nb] = band_here * 32 < pr.N;
    const int band = active[nb] ? band_here : pr.N / 32 - 1;  // past the last band: repeat it, store nothing
    n[nb] = band * 32 + j;
    wband[nb] = pr.wp + (static_cast<int64_t>(band) * (g.K / T::G)) * (P::PIECES * 64) + lane;
  }
  half_t scale_h[NB];  // the columns' int8 scales, requested before the main loop (see stream_block)
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    scale_h[nb] = static_cast<half_t>(1.0f);
    if constexpr (FMT == RWKV_FMT_W8) scale_h[nb] = pr.scale[n[nb]];
  }

  float16_t acc[NB][MT];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[nb][mt][v] = 0.0f;

  constexpr int NK = T::GROUPS * T::STEPS;        // MFMA steps of a chunk
  if constexpr (ROLL) {
    WRegs<FMT, MT, KC> w[NB];
    XRegs<FMT, MT, KC, 4> xq;
    const int last = nchunks - 1;
    xq.request(g, pr, tid, m0, kbeg);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) w[nb].request(g, pr, kbeg, wband[nb], n[nb]);
    xq.store_x(tid, xs);
    __syncthreads();
    static_assert(T::XV % (NK / 2) == 0 && T::STEPS == 2 && T::NW == T::GROUPS,
                  "a whole number of X vectors per MFMA step, two steps per weight piece");
    constexpr int XPS = T::XV / (NK / 2);  // X vectors requested (first half of the steps) or stored (second half) per step
    auto chunk = [&](int u, int c) {
      const half_t* tile = xs + (u & 1) * T::kTileHalfs;
      half_t* tile_next = xs + ((u + 1) & 1) * T::kTileHalfs;
      const int knext = kbeg + (c + 1 <= last ? c + 1 : c) * KC;  // past the end: the current chunk again (in cache)
      const half_t* xlane = tile + j * T::XSTRIDE + h * P::KR;
      half8_t a[2][MT];
      auto load_a = [&](int ks, half8_t (&dst)[MT]) {
        const half_t* xa = xlane + (ks / T::STEPS) * T::G + 8 * (ks % T::STEPS);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) dst[mt] = *reinterpret_cast<const half8_t*>(xa + mt * 32 * T::XSTRIDE);
      };
      load_a(0, a[0]);
#pragma unroll
      for (int ks = 0; ks < NK; ++ks) {
        const int gi = ks / T::STEPS;
        const int st = ks % T::STEPS;
        if (ks + 1 < NK) load_a(ks + 1, a[(ks + 1) & 1]);
#pragma unroll
        for (int i = 0; i < XPS; ++i) {
          if (ks < NK / 2) {
            xq.request_one(XPS * ks + i, g, pr, tid, m0, knext);
          } else {
            xq.store_one(XPS * (ks - NK / 2) + i, tid, tile_next);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const uint4_t piece = w[nb].w[gi];
          const half8_t b = st == 0 ? expand_w8(piece[0], piece[1]) : expand_w8(piece[2], piece[3]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[nb][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks & 1][mt], b, acc[nb][mt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (st == T::STEPS - 1) {  // piece gi has been expanded for the last time: the next chunk's takes its place
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) w[nb].request_piece(gi, knext, wband[nb]);
        }
      }
      __syncthreads();
    };
    const int whole = nchunks - nchunks % 2;
    int c0 = 0;
    for (; c0 < whole; c0 += 2) {
      chunk(0, c0);
      chunk(1, c0 + 1);
    }
    if (c0 < nchunks) chunk(0, c0);
  } else {
  constexpr int D = FMT == RWKV_FMT_F16 ? 2 : 3;  // weight register sets per band
  constexpr int WPS = NB * T::NW / NK;            // weight pieces requested per MFMA step (1 int8, 2 fp16)
  static_assert(T::XV == NK && NB * T::NW % NK == 0, "one X vector and a whole number of weight pieces per MFMA step");
  static_assert(MT == 4, "the ring variant is the 128-row tile");
  WRegs<FMT, MT, KC> wr[D][NB];
  XRegs<FMT, MT, KC, 4> xr[2];
  const int last = nchunks - 1;
  xr[0].request(g, pr, tid, m0, kbeg);
  xr[1].request(g, pr, tid, m0, kbeg + min(1, last) * KC);
#pragma unroll
  for (int i = 0; i < D - 1; ++i)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) wr[i][nb].request(g, pr, kbeg + min(i, last) * KC, wband[nb], n[nb]);
  xr[0].store_x(tid, xs);
  __syncthreads();

  // Chunk c out of LDS tile u & 1 with the weights of ring set u % D.  A wavefront is alone on its SIMD (its 128
  // accumulator registers leave no room for a second one), so whatever it issues besides MFMAs leaves the matrix
  // core idle: the memory work of a chunk is spread over its MFMA steps instead of standing in a block at its
  // head - each step stores one vector of the next chunk's X (requested during the previous chunk) into the other
  // tile, requests one vector of the X of the chunk after that into the register set just freed and WPS pieces of
  // the weights D - 1 chunks ahead.  (Issued in one block, the 16 requests of a chunk took a wavefront 0.5 us of a
  // 2.2 us chunk: four wavefronts queue for the one address unit of the CU.)
  auto chunk = [&](int u, int c) {
    const half_t* tile = xs + (u & 1) * T::kTileHalfs;
    half_t* tile_next = xs + ((u + 1) & 1) * T::kTileHalfs;
    const int kx = kbeg + (c + 2 <= last ? c + 2 : c) * KC;
    const int kw = kbeg + (c + D - 1 <= last ? c + D - 1 : c) * KC;
    const WRegs<FMT, MT, KC> (&w)[NB] = wr[u % D];
    const half_t* xlane = tile + j * T::XSTRIDE + h * P::KR;
    half8_t a[2][MT];
    auto load_a = [&](int ks, half8_t (&dst)[MT]) {
      const half_t* xa = xlane + (ks / T::STEPS) * T::G + 8 * (ks % T::STEPS);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) dst[mt] = *reinterpret_cast<const half8_t*>(xa + mt * 32 * T::XSTRIDE);
    };
    load_a(0, a[0]);
#pragma unroll
    for (int ks = 0; ks < NK; ++ks) {
      const int gi = ks / T::STEPS;
      const int st = ks % T::STEPS;
      if (ks + 1 < NK) load_a(ks + 1, a[(ks + 1) & 1]);
      xr[(u + 1) & 1].store_one(ks, tid, tile_next);
      xr[u & 1].request_one(ks, g, pr, tid, m0, kx);
#pragma unroll
      for (int q = ks * WPS; q < (ks + 1) * WPS; ++q) wr[(u + D - 1) % D][q / T::NW].request_piece(q % T::NW, kw, wband[q / T::NW]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        half8_t b;
        if constexpr (FMT == RWKV_FMT_F16) {
          b = __builtin_bit_cast(half8_t, w[nb].w[gi * 2 + st]);
        } else {
          const uint4_t piece = w[nb].w[gi];
          b = st == 0 ? expand_w8(piece[0], piece[1]) : expand_w8(piece[2], piece[3]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nb][mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks & 1][mt], b, acc[nb][mt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };

  constexpr int U = (D % 2 == 0) ? D : 2 * D;
  // whole rounds of U chunks as one basic block, the chunks left over with exits between them (see stream_block)
  const int whole = nchunks - nchunks % U;
  int c0 = 0;
  for (; c0 < whole; c0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) chunk(u, c0 + u);
  }
  if (c0 < nchunks) {
#pragma unroll
    for (int u = 0; u < U - 1; ++u) {
      if (c0 + u >= nchunks) break;
      chunk(u, c0 + u);
    }
  }
  }  // !ROLL

  // output: one 128-column half of the tile at a time through LDS (the X tiles are free), written in 16/32-byte
  // pieces along the rows
  constexpr int kStageLd = 128 + 8;
  static_assert(BM * kStageLd * 4 <= 2 * T::kTileHalfs * 2, "epilogue tile exceeds the LDS tiles");
  float* stage = reinterpret_cast<float*>(xs);
  const bool partial_out = g.splits > 1;
  float* part_out = partial_out ? pr.partial + static_cast<int64_t>(split) * g.M * pr.N : nullptr;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    if (nb > 0) __syncthreads();  // the previous half has been read
    const float scl = partial_out ? 1.0f : h2f(scale_h[nb]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float sum = acc[nb][mt][v];
        const int row = mt * 32 + 8 * (v >> 2) + 4 * h + (v & 3);
        stage[row * kStageLd + wave * 32 + j] = partial_out ? sum : finish_value(mul_f32(sum, scl), g.epilogue);
      }
    __syncthreads();
    const int col0 = col_block * (128 * NB) + nb * 128;
    for (int idx = tid; idx < BM * 16; idx += 256) {
      const int row = idx >> 4;
      const int piece = idx & 15;
      const int col = col0 + piece * 8;
      if (m0 + row >= g.M || col >= pr.N) continue;
      const float4_t lo = *reinterpret_cast<const float4_t*>(stage + row * kStageLd + piece * 8);
      const float4_t hi = *reinterpret_cast<const float4_t*>(stage + row * kStageLd + piece * 8 + 4);
      const int64_t o = static_cast<int64_t>(m0 + row) * pr.N + col;
      if (partial_out || g.out_f32) {
        float* dst = partial_out ? part_out + o : static_cast<float*>(pr.y) + o;
        *reinterpret_cast<float4_t*>(dst) = lo;
        *reinterpret_cast<float4_t*>(dst + 4) = hi;
      } else {
        half8_t hv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          hv[e] = f2h(lo[e]);
          hv[4 + e] = f2h(hi[e]);
        }
        *reinterpret_cast<half8_t*>(static_cast<half_t*>(pr.y) + o) = hv;
      }
    }
  }
}

// MIXED: the problems of the launch may be int8 or fp16 (one wavefront per SIMD); otherwise all are int8 and two
// blocks share a CU.
template <bool MIXED, int MT>
__global__ __launch_bounds__(256, MIXED ? 1 : 2) void gemm_stream_wide_kernel(StreamArgs g) {
  __shared__ __align__(16) half_t xs[2 * 32 * MT * (128 + 8)];
  ride_along_copy(g.copy);
  const int id = blockIdx.x;
  const int row_tile = (id >> 3) % g.row_tiles;
  const int pair = (id / (8 * g.row_tiles)) * 8 + (id & 7);
  if (pair >= g.col_blocks * g.splits) return;
  const int col_all = pair % g.col_blocks;
  const int split = pair / g.col_blocks;
  int pi = 0;
  while (pi + 1 < g.n_problems && col_all >= g.block_end[pi]) ++pi;
  const int col_block = col_all - (pi > 0 ? g.block_end[pi - 1] : 0);
  const StreamProblem& pr = g.p[pi];
  if constexpr (!MIXED) {
    stream_block_wide<RWKV_FMT_W8, true, MT>(g, pr, row_tile, col_block, split, xs);
  } else if (pr.fmt == RWKV_FMT_W8) {
    stream_block_wide<RWKV_FMT_W8, false, MT>(g, pr, row_tile, col_block, split, xs);
  } else {
    stream_block_wide<RWKV_FMT_F16, false, MT>(g, pr, row_tile, col_block, split, xs);
  }
}

struct ReduceProblem {
  const float4_t* partial;
  const half_t* scale;  // NULL unless the problem's weights are int8 codes
  void* y;
  int N4;
};
struct ReduceArgs {
  ReduceProblem p[kMaxProblems];
  int block_end[kMaxProblems];
  int n_problems;
  int M, splits, epilogue, out_f32;
};

// y = finish(scale * sum over splits of partial), four columns per thread; blocks run over all problems.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(ReduceArgs g) {
  int pi = 0;
  while (pi + 1 < g.n_problems && static_cast<int>(blockIdx.x) >= g.block_end[pi]) ++pi;
  const ReduceProblem& pr = g.p[pi];
  const int64_t plane4 = static_cast<int64_t>(g.M) * pr.N4;
  const int64_t i = static_cast<int64_t>(blockIdx.x - (pi > 0 ? g.block_end[pi - 1] : 0)) * 256 + threadIdx.x;
  if (i >= plane4) return;
  const float4_t* partial = pr.partial;
  // the scale first (without one: any readable vector), then the partials four at a time, each group requested
  // whole before its first member is added, in split order; past the last split the last one is read again and
  // left out - no load waits for an earlier one
  const half4_t sv = *reinterpret_cast<const half4_t*>(pr.scale ? pr.scale + (i % pr.N4) * 4
                                                                : reinterpret_cast<const half_t*>(partial));
  float4_t sum = partial[i];
  for (int base = 1; base < g.splits; base += 4) {
    float4_t q[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) q[u] = partial[(base + u < g.splits ? base + u : g.splits - 1) * plane4 + i];
    // (keeps the four requests together: the compiler would move each load down into the condition of its use)
#pragma unroll
    for (int u = 0; u < 4; ++u) asm volatile("" : "+v"(q[u]));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (base + u < g.splits) sum = sum + q[u];
  }
  float4_t scl = {1.0f, 1.0f, 1.0f, 1.0f};
  if (pr.scale) scl = float4_t{h2f(sv[0]), h2f(sv[1]), h2f(sv[2]), h2f(sv[3])};
  float4_t val;
#pragma unroll
  for (int c = 0; c < 4; ++c) val[c] = finish_value(mul_f32(sum[c], scl[c]), g.epilogue);
  if (g.out_f32) {
    static_cast<float4_t*>(pr.y)[i] = val;
  } else {
    half4_t o;
#pragma unroll
    for (int c = 0; c < 4; ++c) o[c] = f2h(val[c]);
    static_cast<half4_t*>(pr.y)[i] = o;
  }
}

// RWKV_GEMM_BLOCKS (tuning hook) = blocks wanted per launch before K is split.  200 of the 256 CUs: a grid of
// 206 blocks (the r/k/v + LoRA rank-in launch at two row tiles) is 25-30 % faster unsplit than split in two.
static int env_int(const char* name, int fallback) {
  const char* e = getenv(name);
  const int v = e ? atoi(e) : 0;
  return v > 0 ? v : fallback;
}
static int target_blocks() {
  static const int v = env_int("RWKV_GEMM_BLOCKS", 200);
  return v;
}

// Tile per row count (measured on 4096x4096, 16384x4096 and 4096x16384 int8 weights): up to 64 rows one 32-row
// tile per block, so that two or more row tiles share the weights through their XCD's L2 and the split stays
// small; up to 512 rows 64-row tiles; both with two wavefront groups per block.  Above that 128-row tiles with
// one group (128 accumulator registers per lane leave no room for a second wavefront per SIMD).
// 33..64 rows against enough column blocks to occupy the CUs without a K split (the head): one 64-row tile, so that
// no weight is requested by two blocks (268 MB of int8 codes at 64 rows: 95 -> 75 us).
// Up to 32 rows, where 128-column blocks would need a K split: blocks of 64 columns with four groups of two
// wavefronts - twice the blocks per matrix, so half the split (less partial-sum traffic) or none (no reduce
// launch): 16 rows x 16384 columns 23.4 -> 19.6 us; decode steps of 8 / 16 / 32 rows 7 / 5 / 3 % faster.  At 64
// rows the narrow blocks lose (24.5 -> 30 us): every block reads all of X.
// From 385 rows on, int8 and fp16 weights, when 128 x 256 tiles alone give 128 blocks or more: the wide tile, whose
// wavefronts feed two MFMAs from every X fragment they read from LDS and whose blocks request half the X bytes per
// flop (int8 codes, 2048 rows: 16384x4096 436 -> 345 us, 4096x16384 400 -> 317 us; 512 rows x 16384 columns
// 138 -> 104 us).  With fewer blocks it would need a K split where the 64-row tiles need none (512 rows x 4096
// columns: 35 us against 42).  Its registers have no room for the int4 codes' zero points.
constexpr int kWideMinRows = 384, kWideMinBlocks = 128;
struct StreamConfig {
  int mt, kc, kg, wg;
  int nb = 1;  // bands per wavefront
  int cols() const { return 32 * wg * nb; }
};
// (narrow matrices, K up to 2048, take it from 257 rows: at 256 rows x 6656 / 8192 x 2048 the 64 x 128 tiles need
// 19.0 / 19.8 us against 24.5 / 24.9; at 384 rows it is ahead again, 30.2 / 33.4 against 33.9 / 35.1)
bool linear_packed_int8_tile(int M, int K) {
  return M > (K <= 2048 ? 256 : 128) && M <= 1024 && (K <= 4096 || M <= 384);
}

static StreamConfig choose_config(int M, int K, int n_problems, const int* Ns, const int* fmts) {
  int cb128 = 0;
  for (int i = 0; i < n_problems; ++i) cb128 += ceil_div(Ns[i], 128);
  if (M <= 32 && K % (128 * 4) == 0 && cb128 < target_blocks()) {
    // Narrow matrices (K up to 2048) whose 64-column blocks would not fill the chip without a K split: 32-column
    // blocks of one wavefront per K group instead - twice the blocks, half the split or none, and with no split no
    // reduce launch (us with the reduce, 64- / 32-column blocks, 8 rows: 6656 x 2048 11.1 / 9.4, 8192 x 2048
    // 11.4 / 9.9, 2048 x 2048 8.6 / 8.4; at K = 4096 the 64-column blocks win, 4096 x 4096 11.5 / 12.2).
    int cb64 = 0;
    for (int i = 0; i < n_problems; ++i) cb64 += ceil_div(Ns[i], 64);
    if (K <= 2048 && cb64 < target_blocks()) return StreamConfig{1, 128, 4, 1};
    return StreamConfig{1, 128, 4, 2};
  }
  if (M > 32 && M <= 64 && cb128 >= target_blocks()) return StreamConfig{2, 128, 2, 4};
  // 33..64 rows of narrow matrices (K up to 2048): the 64-column blocks again, which here need no K split where the
  // 128-column blocks do, and X is short (us with the reduce, 128- / 64-column blocks, 64 rows: 6656 x 2048
  // 14.0 / 11.5, 8192 x 2048 15.5 / 12.1, 2048 x 2048 10.7 / 9.6)
  if (M > 32 && M <= 64 && K <= 2048 && K % (128 * 4) == 0 && 2 * cb128 < target_blocks()) return StreamConfig{1, 128, 4, 2};
  if (M <= 64) return StreamConfig{1, 128, 2, 4};
  // 65..128 rows against few column blocks (4096 columns and fewer) and a short K: 32-row tiles need half the K
  // split of 64-row tiles for the same number of blocks (128 rows x 4096 x 4096: 19.8 -> 16.6 us; with K = 16384
  // the 64-row tiles win, 35.5 us against 38.1)
  // ... and where the 32-row tiles alone fill the chip and the 64-row tiles do not (128 rows x 6656 x 2048:
  // 19.5 -> 13.4 us, 8192 x 2048: 21.7 -> 14.0; at 96 rows both would split and the 64-row tiles stay ahead)
  if (M <= 128 && K <= 4096 && ceil_div(M, 64) * cb128 < target_blocks() &&
      (ceil_div(M, 64) * cb128 * 2 <= target_blocks() || ceil_div(M, 32) * cb128 >= target_blocks()))
    return StreamConfig{1, 128, 2, 4};
  // 129..1024 rows, int8 weights only, and K up to 4096 or up to 384 rows: the 64 x 256 tile of two bands per
  // wavefront that fits three wavefronts per SIMD (us, 64 x 256 / 128 x 256 / 64 x 128 tiles; * = with a K split:
  // 256 rows x 16384 x 4096 51 / 59* / 64, 384 x 16384 x 4096 74 / 100* / 105, 384 x 4096 x 16384 85* / 96* / 112*,
  // 768 x 12288 x 4096 115 / 139 / 160, 1024 x 4096 x 4096 47 / 56* / 66; against it 512 x 4096 x 16384
  // 108* / 102* / 119 and 1024 x 4096 x 16384 193 / 177* / 223).  Launches with fp16 problems among them keep the
  // tiles below.
  bool all_w8 = true;
  for (int i = 0; i < n_problems; ++i) all_w8 = all_w8 && fmts[i] == RWKV_FMT_W8;
  if (all_w8 && linear_packed_int8_tile(M, K)) return StreamConfig{2, 128, 1, 4, 2};
  // 129..256 rows against enough column blocks: 128-row tiles give one round of blocks where 64-row tiles give
  // two (256 rows x 16384 x 4096: 62.5 -> 56 us)
  if (M > 128 && M <= 256 && 2 * cb128 >= target_blocks() && 2 * cb128 <= 256) return StreamConfig{4, 128, 1, 4};
  bool any_w4 = false;
  int cb256 = 0;
  for (int i = 0; i < n_problems; ++i) {
    any_w4 = any_w4 || fmts[i] == RWKV_FMT_W4;
    cb256 += ceil_div(Ns[i], 256);
  }
  if (M > kWideMinRows && !any_w4 && ceil_div(M, 128) * cb256 >= kWideMinBlocks) return StreamConfig{4, 128, 1, 4, 2};
  if (M <= 512) return StreamConfig{2, 128, 2, 4};
  return StreamConfig{4, 128, 1, 4};
}
static int count_col_blocks(const StreamConfig& c, int n_problems, const int* Ns) {
  int col_blocks = 0;
  for (int i = 0; i < n_problems; ++i) col_blocks += ceil_div(Ns[i], c.cols());
  return col_blocks;
}

// Split count: a power of two that gives enough blocks to occupy the CUs, K slices whole chunks of every group.
static int choose_splits(const StreamConfig& c, int M, int col_blocks, int K) {
  const int tiles = ceil_div(M, 32 * c.mt) * col_blocks;
  int splits = 1;
  while (tiles * splits < target_blocks() && K % (splits * 2 * c.kc * c.kg) == 0 && splits < 32) splits *= 2;
  return splits;
}

// The formats are not known here: the larger of what the tiles with and without int4 weights would need.
size_t linear_packed_multi_workspace_bytes(int M, int K, int n_problems, const int* Ns) {
  int64_t n_total = 0;
  for (int i = 0; i < n_problems; ++i) n_total += Ns[i];
  int fmts[kMaxProblems];
  size_t need = 0;
  for (int fmt : {RWKV_FMT_W8, RWKV_FMT_W4, RWKV_FMT_F16}) {  // all int8, some int4, neither (fp16 among them)
    for (int i = 0; i < n_problems && i < kMaxProblems; ++i) fmts[i] = fmt;
    const StreamConfig c = choose_config(M, K, n_problems, Ns, fmts);
    const int splits = choose_splits(c, M, count_col_blocks(c, n_problems, Ns), K);
    if (splits > 1) need = std::max(need, static_cast<size_t>(splits) * M * n_total * sizeof(float));
  }
  return need;
}

size_t linear_packed_workspace_bytes(int M, int N, int K) { return linear_packed_multi_workspace_bytes(M, K, 1, &N); }

int linear_packed_multi(hipStream_t st, int M, int K, int n_problems, const PackedProblem* problems, int epilogue,
                        int out_f32, void* workspace, size_t workspace_bytes, DeferredReduce* defer, const RowCopy* copy) {
  RWKV_REQUIRE(n_problems >= 1 && n_problems <= kMaxProblems, "linear_packed: %d problems (1..%d allowed)", n_problems,
               kMaxProblems);
  StreamArgs g;
  ReduceArgs r;
  if (copy) {
    RWKV_REQUIRE(copy->n >= 0 && copy->n % 8 == 0 && (copy->n == 0 || (copy->src && copy->dst)), "linear_packed: bad row copy");
    g.copy = *copy;
  }
  g.n_problems = r.n_problems = n_problems;
  g.M = r.M = M;
  g.K = K;
  g.epilogue = r.epilogue = epilogue;
  g.out_f32 = r.out_f32 = out_f32;
  int Ns[kMaxProblems], fmts[kMaxProblems];
  for (int i = 0; i < n_problems; ++i) {
    Ns[i] = problems[i].N;
    fmts[i] = problems[i].fmt;
  }
  const StreamConfig cfg = choose_config(M, K, n_problems, Ns, fmts);
  int col_blocks = 0;
  for (int i = 0; i < n_problems; ++i) {
    const PackedProblem& q = problems[i];
    RWKV_REQUIRE(linear_packed_supported(q.fmt, M, q.N, K), "linear_packed: unsupported shape M=%d N=%d K=%d fmt=%d", M,
                 q.N, K, q.fmt);
    RWKV_REQUIRE(q.x && q.packed && q.y, "linear_packed: NULL tensor");
    RWKV_REQUIRE(q.fmt == RWKV_FMT_F16 || q.scale, "linear_packed: quantised weights need a scale tensor");
    RWKV_REQUIRE(q.fmt != RWKV_FMT_W4 || q.zp, "linear_packed: W4 weights need a zero-point tensor");
    col_blocks += ceil_div(q.N, cfg.cols());
    g.block_end[i] = col_blocks;
    g.p[i] = StreamProblem{q.x, static_cast<const uint4_t*>(q.packed), q.scale, q.zp, q.y, nullptr, q.N, q.fmt};
  }
  g.splits = r.splits = choose_splits(cfg, M, col_blocks, K);
  g.k_per_split = K / g.splits;
  if (g.splits > 1) {
    size_t need = 0;
    for (int i = 0; i < n_problems; ++i) need += static_cast<size_t>(g.splits) * M * problems[i].N * sizeof(float);
    RWKV_REQUIRE(workspace && workspace_bytes >= need, "linear_packed: workspace of %zu bytes needed, got %zu", need,
                 workspace_bytes);
    float* at = static_cast<float*>(workspace);
    int red_blocks = 0;
    for (int i = 0; i < n_problems; ++i) {
      g.p[i].partial = at;
      const int64_t plane4 = static_cast<int64_t>(M) * problems[i].N / 4;
      red_blocks += static_cast<int>((plane4 + 255) / 256);
      r.block_end[i] = red_blocks;
      r.p[i] = ReduceProblem{reinterpret_cast<const float4_t*>(at),
                             problems[i].fmt == RWKV_FMT_W8 ? problems[i].scale : nullptr, problems[i].y, problems[i].N / 4};
      at += static_cast<size_t>(g.splits) * M * problems[i].N;
    }
  }
  RWKV_REQUIRE(g.k_per_split % (cfg.kc * cfg.kg) == 0, "linear_packed: K slice %d is not a whole number of %d-chunks",
               g.k_per_split, cfg.kc * cfg.kg);
  g.row_tiles = ceil_div(M, 32 * cfg.mt);
  g.col_blocks = col_blocks;
  const int pairs8 = ceil_div(col_blocks * g.splits, 8) * 8;
  const dim3 grid(g.row_tiles * pairs8);
  const dim3 block(64 * cfg.wg * cfg.kg);
  bool all_w8 = true;
  for (int i = 0; i < n_problems; ++i) all_w8 = all_w8 && problems[i].fmt == RWKV_FMT_W8;
  if (cfg.nb == 2 && cfg.mt == 2) {
    RWKV_REQUIRE(all_w8, "linear_packed: the 64 x 256 tile takes int8 weights only");
    hipLaunchKernelGGL((gemm_stream_wide_kernel<false, 2>), grid, block, 0, st, g);
  } else if (cfg.nb == 2) hipLaunchKernelGGL((gemm_stream_wide_kernel<true, 4>), grid, block, 0, st, g);
  else if (cfg.wg == 1) hipLaunchKernelGGL((gemm_stream_kernel<1, 128, 4, 1>), grid, block, 0, st, g);
  else if (cfg.wg == 2) hipLaunchKernelGGL((gemm_stream_kernel<1, 128, 4, 2>), grid, block, 0, st, g);
  else if (cfg.mt == 1) hipLaunchKernelGGL((gemm_stream_kernel<1, 128, 2, 4>), grid, block, 0, st, g);
  else if (cfg.mt == 2) hipLaunchKernelGGL((gemm_stream_kernel<2, 128, 2, 4>), grid, block, 0, st, g);
  else hipLaunchKernelGGL((gemm_stream_kernel<4, 128, 1, 4>), grid, block, 0, st, g);
  RWKV_LAUNCH_CHECK();
  if (defer) *defer = DeferredReduce{};
  if (g.splits == 1) return RWKV_OK;
  if (defer) {
    RWKV_REQUIRE(n_problems == 1 && epilogue == RWKV_EPI_NONE && !out_f32,
                 "linear_packed: a deferred reduce takes one problem, fp16 output and no epilogue");
    defer->partial = g.p[0].partial;
    defer->scale = problems[0].fmt == RWKV_FMT_W8 ? problems[0].scale : nullptr;
    defer->plane = static_cast<int64_t>(M) * problems[0].N;
    defer->splits = g.splits;
    return RWKV_OK;
  }
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3(r.block_end[n_problems - 1]), dim3(256), 0, st, r);
  RWKV_LAUNCH_CHECK();
  return RWKV_OK;
}

int linear_packed(hipStream_t st, int fmt, int M, int N, int K, const half_t* x, const void* packed, const half_t* scale,
                  const uint8_t* zp, int epilogue, int out_f32, void* y, void* workspace, size_t workspace_bytes,
                  DeferredReduce* defer, const RowCopy* copy) {
  const PackedProblem q = {packed, scale, zp, x, y, N, fmt};
  return linear_packed_multi(st, M, K, 1, &q, epilogue, out_f32, workspace, workspace_bytes, defer, copy);
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_hip_pack_weights(rwkv_stream_t s, int fmt, int N, int K, const void* w, void* packed) {
  return pack_weights_launch(as_stream(s), fmt, N, K, w, packed);
}

int rwkv_hip_linear_packed_workspace(int M, int N, int K, size_t* bytes) {
  RWKV_REQUIRE(bytes && M > 0 && N > 0 && K > 0, "linear_packed_workspace: bad arguments");
  *bytes = linear_packed_workspace_bytes(M, N, K);
  return RWKV_OK;
}

int rwkv_hip_linear_packed(rwkv_stream_t s, int fmt, int M, int N, int K, const void* x, const void* packed,
                           const void* scale, const void* zp, int epilogue, int out_f32, void* y, void* workspace,
                           size_t workspace_bytes) {
  RWKV_REQUIRE(epilogue == RWKV_EPI_NONE || epilogue == RWKV_EPI_RELU_SQUARE, "linear_packed: bad epilogue %d", epilogue);
  return linear_packed(as_stream(s), fmt, M, N, K, static_cast<const half_t*>(x), packed,
                       static_cast<const half_t*>(scale), static_cast<const uint8_t*>(zp), epilogue, out_f32, y, workspace,
                       workspace_bytes);
}

}  // extern "C"
