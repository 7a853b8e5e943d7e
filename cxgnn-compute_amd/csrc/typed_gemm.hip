// Typed (relation-segmented) GEMM on the gfx950 matrix cores:
//
//   C[dst(i), :] (=, +=, atomic +=)  A[src(i), :] @ W[rel(i)],   i in [0, M)
//
// Rows are grouped by relation: rows seg[r] .. seg[r+1]-1 use W[r].  A tile of 64
// rows never crosses a segment; the tail of a segment is masked instead of
// padded (the reference pads every relation up to a multiple of the tile with
// sentinel rows, cxgnncomp/typed_linear.py:74-87, src/cpp/src/stitch_kernel.cu).
// src / dst are optional row maps (gather of A rows, scatter of C rows); a
// negative entry skips the row -- that is how the reference's padded layout is
// accepted unchanged.
//
// This is the only dense contraction of the library and the only MFMA user:
//   fp32:  v_mfma_f32_32x32x2_f32     (A, W fp32 in memory)
//   bf16:  v_mfma_f32_32x32x16_bf16   (A bf16, W^T bf16 in memory, fp32 accumulate/out)
// Block = 4 waves, tile 64 x BN (BN = 128 or 64), K walked in LDS chunks that
// are double-buffered against the global loads of the next chunk.
//
// Replaces the Triton typed_matmul kernels
// (cxgnncomp/codegen/triton_typed_matmul.py:146-215,364-430,529-592,691-749;
// launcher :752-860) and, through the host wrappers, the per-row CUDA kernels
// typed_linear_kernel / _s2e / _s2d (src/cpp/src/rel_spmm.cu:231-358).
#include <type_traits>

#include "cxg_common.hpp"
#include "split_f16.hpp"

namespace cxg {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

constexpr int kBM = 64;
constexpr int kThreads = 256;
constexpr int kXcds = 8;                 // accelerator dies of an MI355X, one L2 each

struct GemmArgs {
  const void* a;
  int64_t lda;
  const void* w;
  float* c;
  int64_t ldc;
  const int64_t* src;
  const int64_t* dst;
  const int64_t* seg;
  int64_t M;
  int K, N, R;
  int accumulate, atomic;
  // epilogue of the split kernel: C[d, n] = (A W)[., n] + bias[r, n] + addend[d, n] (either may be null)
  const float* bias;
  const float* addend;
  int64_t ldd;
  int c_bf16;             // the rows of C are bf16 (ldc in elements): the bf16-operand kernels, plain stores only
};

// Tile number -> (relation, first row, end of the relation's rows).  Every thread
// walks the R+1 segment offsets; the result is block-uniform.
__device__ __forceinline__ bool locate_tile(const int64_t* __restrict__ seg, int R, int64_t tile,
                                            int& rel, int64_t& row0, int64_t& row_end) {
  int64_t t = tile;
  for (int r = 0; r < R; ++r) {
    const int64_t b = seg[r], e = seg[r + 1];
    const int64_t nt = (e - b + kBM - 1) / kBM;
    if (t < nt) {
      rel = r;
      row0 = b + t * kBM;
      row_end = e;
      return true;
    }
    t -= nt;
  }
  return false;
}

// Output of one block tile.  In the 32x32 MFMA accumulator a lane holds, for its column,
// four groups of four consecutive rows; the destination rows of a group are fetched from
// LDS together (they are 32 contiguous bytes) and the four stores follow without waits.
// MODE 0: store, 1: read-add-store, 2: fp32 atomic add.
template <int BN, int MT, int MODE, bool EPI = false, int QB = 1>
__device__ __forceinline__ void store_tile_mode(const GemmArgs& g, const v16f (&acc)[MT],
                                                const int64_t* s_dst, int wm, int wn, int lane, int n0) {
  const int col = n0 + wn * 32 + (lane & 31);
  if (col >= g.N) return;
  float* const base = g.c + col;
  const int64_t ldc = g.ldc;
  if (MODE != 1 && !(EPI && g.addend)) {
    // nothing is read: the rows of a group of four as soon as their indices are there
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int rl0 = (wm * MT + mt) * 32 + q * 8 + (lane >> 5) * 4;
        int64_t d[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) d[j] = s_dst[rl0 + j];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (d[j] < 0) continue;
          float* p = base + d[j] * ldc;
          if (MODE == 2) unsafeAtomicAdd(p, acc[mt][q * 4 + j]);
          else *p = acc[mt][q * 4 + j];
        }
      }
    }
    return;
  }
  if constexpr (QB == 4 && MODE == 1) {
    // Accumulation: the old rows of the whole tile are requested first, then all sums are
    // formed, then all rows are stored (with an addend only, 16 rows at a time as below
    // measured faster: 2.45 M x 256 x 256 2.92 against 3.23 ms; accumulation 3.21 -> 2.73 ms).  Loads and stores of
    // a wave share one in-order counter and a store may be acknowledged before an older load
    // returns, so a load that is waited for after a store is waited for together with that
    // store's acknowledgement; and a read-add-store per element in turn is one trip to memory
    // after the other, since a store may alias the next load.  The loads carry no condition
    // (rows that do not exist read a weight element instead); the row indices are read from
    // LDS a second time for the stores rather than kept.
    float o[MT][16];
    const bool both = EPI && g.addend;
    const float* const src = both ? g.addend + col : base;
    const int64_t ld = both ? g.ldd : ldc;
    const float* const safe = reinterpret_cast<const float*>(g.w) + col;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int rl0 = (wm * MT + mt) * 32 + q * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t d = s_dst[rl0 + j];
          o[mt][q * 4 + j] = *(d >= 0 ? src + d * ld : safe);
        }
      }
    if (both) {                              // accumulation and an addend: the old rows as well
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int rl0 = (wm * MT + mt) * 32 + q * 8 + (lane >> 5) * 4;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int64_t d = s_dst[rl0 + j];
            o[mt][q * 4 + j] += *(d >= 0 ? base + d * ldc : safe);
          }
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        o[mt][i] += acc[mt][i];
        asm volatile("" : "+v"(o[mt][i]));   // (an opaque use: otherwise each sum moves down to its store)
      }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int rl0 = (wm * MT + mt) * 32 + q * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t d = s_dst[rl0 + j];
          if (d >= 0) base[d * ldc] = o[mt][q * 4 + j];
        }
      }
    return;
  }
  // What the rows are added to (the old row when accumulating, the addend) is requested for
  // 4 * QB rows before their first store: a read-add-store per element in turn is one trip
  // to memory after the other, since a store may alias the next load.
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int q0 = 0; q0 < 4; q0 += QB) {
      constexpr int NR = 4 * QB;
      int64_t d[NR];
      float v[NR];
#pragma unroll
      for (int q = 0; q < QB; ++q) {
        const int rl0 = (wm * MT + mt) * 32 + (q0 + q) * 8 + (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          d[q * 4 + j] = s_dst[rl0 + j];
          v[q * 4 + j] = acc[mt][(q0 + q) * 4 + j];
        }
      }
      if (MODE == 1) {
        float o[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) o[i] = d[i] >= 0 ? base[d[i] * ldc] : 0.f;
#pragma unroll
        for (int i = 0; i < NR; ++i) v[i] += o[i];
      }
      if (EPI && g.addend) {
        float o[NR];
#pragma unroll
        for (int i = 0; i < NR; ++i) o[i] = d[i] >= 0 ? g.addend[d[i] * g.ldd + col] : 0.f;
#pragma unroll
        for (int i = 0; i < NR; ++i) v[i] += o[i];
      }
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        if (d[i] < 0) continue;
        float* p = base + d[i] * ldc;
        if (MODE == 2) unsafeAtomicAdd(p, v[i]);
        else *p = v[i];
      }
    }
  }
}

// bf16 rows of C (N and ldc even, plain stores).  A lane holds four consecutive rows of ONE
// column; it swaps values with the lane of the neighbouring column (lane ^ 1) so that the even
// lane stores rows 0 and 1 and the odd lane rows 2 and 3 of each group as pairs of columns:
// 4-byte stores instead of 2-byte ones.
template <int MT>
__device__ __forceinline__ void store_tile_bf16(const GemmArgs& g, const v16f (&acc)[MT], const int64_t* s_dst, int wn,
                                                int lane, int n0) {
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  const int col = n0 + wn * 32 + (lane & 31);
  const bool odd = lane & 1;
  uint16_t* const base = reinterpret_cast<uint16_t*>(g.c) + (col & ~1);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int rl0 = mt * 32 + q * 8 + (lane >> 5) * 4;
      float other[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        other[j] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc[mt][q * 4 + j]), 0xB1, 0xf, 0xf, false));
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int j = odd ? 2 + h : h;
        const float mine = acc[mt][q * 4 + j], theirs = other[j];
        const v2bf pr = {(__bf16)(odd ? theirs : mine), (__bf16)(odd ? mine : theirs)};
        const int64_t d = s_dst[rl0 + j];
        if (d >= 0 && col < g.N) *reinterpret_cast<unsigned*>(base + d * g.ldc) = __builtin_bit_cast(unsigned, pr);
      }
    }
  }
}

// The same rows through a per-wave LDS area of 32 rows x 32 columns (80-byte pitch), one 32 x 32
// accumulator block at a time: the pairs of columns are written as 4-byte words, read back as 16
// bytes per lane -- four lanes per row, sixteen rows per instruction -- and stored as such: four
// store instructions per tile and wave instead of sixteen, each writing 64 contiguous bytes of
// sixteen rows.  (8.2 M rows x 128 x 128, bf16 in and out: 1.40 ms, of which 0.85 ms were the 4-byte
// stores -- the kernel without them took 0.55 ms.)  The wave's LDS operations execute in order, so
// the area needs no barrier.  For whole 32-column pieces and 16-byte aligned rows.
constexpr int kCsPitch = 40;                 // bf16 elements per staged row
template <int MT>
__device__ __forceinline__ void store_tile_bf16_staged(const GemmArgs& g, const v16f (&acc)[MT], const int64_t* s_dst,
                                                       int wn, int lane, int n0, uint16_t* cs) {
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  const bool odd = lane & 1;
  uint16_t* const base = reinterpret_cast<uint16_t*>(g.c) + n0 + wn * 32 + (lane & 3) * 8;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float other[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        other[j] = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc[mt][q * 4 + j]), 0xB1, 0xf, 0xf, false));
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int j = odd ? 2 + h : h;
        const float mine = acc[mt][q * 4 + j], theirs = other[j];
        const v2bf pr = {(__bf16)(odd ? theirs : mine), (__bf16)(odd ? mine : theirs)};
        const int row = q * 8 + (lane >> 5) * 4 + j;
        *reinterpret_cast<unsigned*>(cs + row * kCsPitch + ((lane & 31) & ~1)) = __builtin_bit_cast(unsigned, pr);
      }
    }
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int row = it * 16 + (lane >> 2);
      const v4u piece = *reinterpret_cast<const v4u*>(cs + row * kCsPitch + (lane & 3) * 8);
      const int64_t d = s_dst[mt * 32 + row];
      if (d >= 0) *reinterpret_cast<v4u*>(base + d * g.ldc) = piece;
    }
  }
}

template <int BN, int MT, bool EPI = false, int QB = 1>
__device__ __forceinline__ void store_tile(const GemmArgs& g, const v16f (&acc)[MT],
                                           const int64_t* s_dst, int wm, int wn, int lane, int n0) {
  if (g.atomic) store_tile_mode<BN, MT, 2, EPI, QB>(g, acc, s_dst, wm, wn, lane, n0);
  else if (g.accumulate) store_tile_mode<BN, MT, 1, EPI, QB>(g, acc, s_dst, wm, wn, lane, n0);
  else store_tile_mode<BN, MT, 0, EPI, QB>(g, acc, s_dst, wm, wn, lane, n0);
}

__device__ __forceinline__ void load_row_maps(const GemmArgs& g, int64_t row0, int64_t row_end,
                                              int64_t* s_src, int64_t* s_dst, int tid) {
  if (tid < kBM) {
    const int64_t gr = row0 + tid;
    int64_t s = -1, d = -1;
    if (gr < row_end) {
      s = g.src ? g.src[gr] : gr;
      d = g.dst ? g.dst[gr] : gr;
      if (s < 0 || d < 0) { s = -1; d = -1; }
    }
    s_src[tid] = s;
    s_dst[tid] = d;
  }
}

// ----------------------------------------------------------------------------
// fp32
// ----------------------------------------------------------------------------
template <int BN>
__global__ __launch_bounds__(kThreads) void typed_gemm_f32_kernel(GemmArgs g) {
  constexpr int KC = 32;
  constexpr int WN = BN / 32, WM = 4 / WN, MT = 2 / WM;
  constexpr int WPT = BN * KC / kThreads;      // W elements per thread per chunk
  __shared__ float As[2][kBM][KC + 1];
  __shared__ float Ws[2][KC][BN];
  __shared__ __attribute__((aligned(16))) int64_t s_src[kBM], s_dst[kBM];
  int rel = 0;
  int64_t row0 = 0, row_end = 0;
  if (!locate_tile(g.seg, g.R, blockIdx.x, rel, row0, row_end)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int n0 = blockIdx.y * BN;
  const int K = g.K, N = g.N;
  load_row_maps(g, row0, row_end, s_src, s_dst, tid);
  __syncthreads();
  const float* W = reinterpret_cast<const float*>(g.w) + (int64_t)rel * K * N;
  const int arow = tid >> 2, akq = (tid & 3) * 8;
  const int64_t asrc = s_src[arow];
  const float* aptr = asrc >= 0 ? reinterpret_cast<const float*>(g.a) + asrc * g.lda : nullptr;
  const bool a_vec = ((g.lda & 3) == 0) && ((reinterpret_cast<uintptr_t>(g.a) & 15) == 0) && ((K & 3) == 0);
  float areg[8], wreg[WPT];
  auto gload = [&](int k0) {
    if (aptr && a_vec) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const int k = k0 + akq + 4 * q;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < K) v = *reinterpret_cast<const float4*>(aptr + k);
        areg[4 * q] = v.x; areg[4 * q + 1] = v.y; areg[4 * q + 2] = v.z; areg[4 * q + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + akq + j;
        areg[j] = (aptr && k < K) ? aptr[k] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      const int e = tid + kThreads * j;
      const int kk = k0 + e / BN, nn = n0 + e % BN;
      wreg[j] = (kk < K && nn < N) ? W[(int64_t)kk * N + nn] : 0.f;
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 8; ++j) As[buf][arow][akq + j] = areg[j];
#pragma unroll
    for (int j = 0; j < WPT; ++j) {
      const int e = tid + kThreads * j;
      Ws[buf][e / BN][e % BN] = wreg[j];
    }
  };
  v16f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;

  const int nchunks = (K + KC - 1) / KC;
  gload(0);
  sstore(0);
  __syncthreads();
  for (int c = 0; c < nchunks; ++c) {
    const int buf = c & 1;
    if (c + 1 < nchunks) gload((c + 1) * KC);
#pragma unroll
    for (int kk = 0; kk < KC; kk += 2) {
      const float b = Ws[buf][kk + (lane >> 5)][wn * 32 + (lane & 31)];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const float a = As[buf][(wm * MT + mt) * 32 + (lane & 31)][kk + (lane >> 5)];
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[mt], 0, 0, 0);
      }
    }
    if (c + 1 < nchunks) sstore(buf ^ 1);
    __syncthreads();
  }
  store_tile<BN, MT>(g, acc, s_dst, wm, wn, lane, n0);
}

// ----------------------------------------------------------------------------
// bf16 inputs (A [*, K] bf16, W^T [R, N, K] bf16), fp32 accumulate and output
// ----------------------------------------------------------------------------
template <int BN>
__global__ __launch_bounds__(kThreads) void typed_gemm_bf16_kernel(GemmArgs g) {
  constexpr int KC = 64;                      // bf16 elements per chunk (128 B per row)
  constexpr int LD = KC + 8;                  // padded LDS row (elements)
  constexpr int WN = BN / 32, WM = 4 / WN, MT = 2 / WM;
  constexpr int WV = BN * KC / 8 / kThreads;  // 16-byte W vectors per thread per chunk
  __shared__ __attribute__((aligned(16))) uint16_t As[2][kBM][LD];
  __shared__ __attribute__((aligned(16))) uint16_t Wt[2][BN][LD];
  __shared__ __attribute__((aligned(16))) int64_t s_src[kBM], s_dst[kBM];
  int rel = 0;
  int64_t row0 = 0, row_end = 0;
  if (!locate_tile(g.seg, g.R, blockIdx.x, rel, row0, row_end)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int n0 = blockIdx.y * BN;
  const int K = g.K, N = g.N;
  load_row_maps(g, row0, row_end, s_src, s_dst, tid);
  __syncthreads();
  const uint16_t* W = reinterpret_cast<const uint16_t*>(g.w) + (int64_t)rel * N * K;
  const int arow = tid >> 2, akq = (tid & 3) * 16;
  const int64_t asrc = s_src[arow];
  const uint16_t* aptr = asrc >= 0 ? reinterpret_cast<const uint16_t*>(g.a) + asrc * g.lda : nullptr;
  uint4 areg[2], wreg[WV];
  const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
  auto gload = [&](int k0) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int k = k0 + akq + 8 * q;
      areg[q] = (aptr && k < K) ? *reinterpret_cast<const uint4*>(aptr + k) : zero4;
    }
#pragma unroll
    for (int j = 0; j < WV; ++j) {
      const int e = tid + kThreads * j;
      const int nn = n0 + e / 8, k = k0 + (e % 8) * 8;
      wreg[j] = (nn < N && k < K) ? *reinterpret_cast<const uint4*>(W + (int64_t)nn * K + k) : zero4;
    }
  };
  auto sstore = [&](int buf) {
#pragma unroll
    for (int q = 0; q < 2; ++q) *reinterpret_cast<uint4*>(&As[buf][arow][akq + 8 * q]) = areg[q];
#pragma unroll
    for (int j = 0; j < WV; ++j) {
      const int e = tid + kThreads * j;
      *reinterpret_cast<uint4*>(&Wt[buf][e / 8][(e % 8) * 8]) = wreg[j];
    }
  };
  v16f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;

  const int nchunks = (K + KC - 1) / KC;
  gload(0);
  sstore(0);
  __syncthreads();
  for (int c = 0; c < nchunks; ++c) {
    const int buf = c & 1;
    if (c + 1 < nchunks) gload((c + 1) * KC);
#pragma unroll
    for (int kk = 0; kk < KC; kk += 16) {
      const v8bf b = *reinterpret_cast<const v8bf*>(&Wt[buf][wn * 32 + (lane & 31)][kk + (lane >> 5) * 8]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const v8bf a = *reinterpret_cast<const v8bf*>(
            &As[buf][(wm * MT + mt) * 32 + (lane & 31)][kk + (lane >> 5) * 8]);
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[mt], 0, 0, 0);
      }
    }
    if (c + 1 < nchunks) sstore(buf ^ 1);
    __syncthreads();
  }
  store_tile<BN, MT>(g, acc, s_dst, wm, wn, lane, n0);
}

// ----------------------------------------------------------------------------
// fp32 operands, products on the bf16 matrix cores as partial products
// ----------------------------------------------------------------------------
// x = p0 + p1 (+ p2) with p0 = bf16(x), p1 = bf16(x - p0), p2 = bf16(x - p0 - p1):
// NS parts keep 8*NS significant bits of each operand.  a*b is accumulated in fp32
// from the partial products a_i*b_j with i + j < NS, smallest first:
//   NS = 3: six products, every dropped term is below 2^-24 |ab| -- the result is
//           as accurate as an fp32 FMA chain;
//   NS = 2: three products, relative error per product below 2^-16 (the TF32
//           tl.dot of the reference's Triton kernel is 2^-11).
// Six bf16 MFMAs take 3/8 of the cycles of the fp32 MFMA for the same K, which
// turns the K, N <= 128 typed GEMM from matrix-core bound into HBM bound.
//
// A block owns up to G consecutive 64-row tiles of ONE relation and has two kinds of
// waves.  The four consumer waves keep the relation's weight slab in registers, already
// split and in MFMA operand layout (wave w: columns 32w..32w+31), so W is fetched once
// per 64*G rows; they multiply a tile out of LDS and store it.  The four producer waves
// fetch the A rows as 16-byte-per-lane row segments, split them into their bf16 parts
// and write the parts of the NEXT tile into the other half of a double-buffered LDS
// area while the consumers multiply.  One barrier per tile separates the two halves.
//
// Why two kinds of waves: a wave's memory counter completes in order, so a wave that
// both loads and stores cannot wait for a load without also waiting for every store it
// issued before it -- the stores of a tile then have to drain (microseconds under a
// write-heavy load) before the next tile can be staged.  Consumer waves never wait on
// memory: their stores (or atomics) stay in flight for as long as the hardware queue
// allows (when rows are added to -- accumulation, an addend -- they wait once per tile,
// for old rows requested a tile earlier; see the tile loops).  Producer waves only ever
// wait for their own loads.  The conversion work of
// the producers runs on the same SIMDs in the shadow of the consumers' MFMAs.
template <int NS>
__device__ __forceinline__ void split_bf16(float x, __bf16 (&p)[NS]) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    p[i] = (__bf16)x;
    x -= (float)p[i];
  }
}

// Scaled fp16 parts (F16): every A row and every W column is scaled by a power of two that
// brings its largest magnitude into [2^14, 2^15) and split into TWO fp16 parts,
// h0 = fp16(x s), h1 = fp16(x s - h0): 22 significant bits.  a*b is accumulated from
// a0*b1, a1*b0, a0*b0 (the dropped a1*b1 is below 2^-22 |ab|) on v_mfma_f32_32x32x16_f16,
// and the accumulator is multiplied by the two inverse scales when the tile is stored.
// Three matrix instructions and two LDS parts per k-step instead of six and three, at
// 2^-21 per product (fp32 itself rounds every product to 2^-24).  The matrix instruction
// keeps fp16 subnormals, so an element keeps its 22 bits down to 2^-17 of its row's
// maximum and is off by at most 2^-39 of that maximum below -- invisible next to the
// rounding of the larger terms of the same dot product.  bf16 has no such range limit
// but only 8 bits per part.
//
// scale 2^(14 - e) and its inverse for a maximum with biased exponent `eb` (e = eb - 127);
// all-zero (or denormal) rows / columns get scale 0, rows with an infinity or NaN scale 1.
__device__ __forceinline__ void pow2_scales(unsigned max_bits, float& scale, float& inv) {
  const int eb = (int)(max_bits >> 23);
  scale = 0.f;
  inv = 0.f;
  if (eb == 255) {
    scale = 1.f;
    inv = 1.f;
  } else if (eb >= 15) {
    scale = __uint_as_float((unsigned)(268 - eb) << 23);
    inv = __uint_as_float((unsigned)(eb - 14) << 23);
  }
}

// Largest value over the aligned group of LANES lanes (8, 16 or 32) that holds a row, in every
// lane of the group: butterfly steps through data-parallel moves inside a 16-lane row (lane ^ 1,
// lane ^ 2, mirror of the row's halves, mirror of the row) and one swizzle for lane ^ 16.
template <int CTRL>
__device__ __forceinline__ unsigned dpp_max_u32(unsigned m) {
  const unsigned o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)m, CTRL, 0xf, 0xf, false);
  return o > m ? o : m;
}
template <int LANES>
__device__ __forceinline__ unsigned group_max_u32(unsigned m) {
  m = dpp_max_u32<0xB1>(m);                  // quad_perm [1,0,3,2]
  m = dpp_max_u32<0x4E>(m);                  // quad_perm [2,3,0,1]
  m = dpp_max_u32<0x141>(m);                 // row_half_mirror
  if (LANES >= 16) m = dpp_max_u32<0x140>(m);   // row_mirror
  if (LANES >= 32) {
    const unsigned o = (unsigned)__builtin_amdgcn_ds_swizzle((int)m, 0x401F);   // lane ^ 16
    m = o > m ? o : m;
  }
  if (LANES >= 64) {
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)m, 0), hi = (unsigned)__builtin_amdgcn_readlane((int)m, 32);
    m = lo > hi ? lo : hi;
  }
  return m;
}

constexpr int kSplitThreads = 512;         // waves 0-3 consume, waves 4-7 produce
constexpr int kMapSlots = 8;               // no row maps given: the row tables of tiles t-1 .. t+5 are live at once
constexpr int kMappedTiles = 16;           // row maps given: a block keeps the maps of ALL its tiles in LDS, so it
                                           // owns at most this many tiles
constexpr int kCP = 40;                    // floats per staged output row: 32 + pad; rows r and
                                           // r + 4 (the two halves of a wave) land 32 banks apart

// EPI: bias and addend of GemmArgs are honoured (a separate instantiation: the extra loads and
// adds in the consumers' loop cost the plain form a tenth of its speed otherwise).
template <int KS, int NS, bool MAPPED, bool F16, bool EPI = false>
__global__ __launch_bounds__(kSplitThreads) __attribute__((amdgpu_waves_per_eu(2)))
void typed_gemm_split_kernel(GemmArgs g, int G) {
  static_assert(!F16 || NS == 2, "the fp16 form has two parts");
  constexpr int KP = KS * 16 + 8;          // padded LDS row (bf16 elements)
  constexpr int LPR = KS * 4;              // lanes per A row, one float4 each
  constexpr int RPI = 256 / LPR;           // rows per load instruction (256 producer threads)
  constexpr int NLD = kBM / RPI;           // load instructions per tile
  typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int SLOTS = MAPPED ? kMappedTiles : kMapSlots;
  // layout: Ap[2][NS][kBM][KP] bf16, s_src / s_dst [SLOTS][kBM] int64, then one
  // [kBM][kCP] fp32 staging area per consumer wave for its 64 x 32 piece of the output
  uint16_t (*Ap)[NS][kBM][KP] = reinterpret_cast<uint16_t (*)[NS][kBM][KP]>(smem);
  int64_t (*s_src)[kBM] = reinterpret_cast<int64_t (*)[kBM]>(smem + sizeof(uint16_t) * 2 * NS * kBM * KP);
  int64_t (*s_dst)[kBM] = s_src + SLOTS;
  // F16: inverse row scales of the two staged tiles, [2][kBM] floats; then the staging areas (the
  // widest form, KS = 16, has no room for them and stores from the accumulators)
  float (*s_inv)[kBM] = reinterpret_cast<float (*)[kBM]>(s_dst + SLOTS);
  float (*Cw)[kCP] = reinterpret_cast<float (*)[kCP]>(reinterpret_cast<unsigned char*>(s_inv + 2)) +
                     (size_t)(threadIdx.x >> 6 & 3) * kBM;
  const int64_t span = (int64_t)kBM * G;
  int rel = -1;
  int64_t row0 = 0, row_end = 0;
  // Blocks are handed to the 8 XCDs round-robin by block index and every XCD has
  // its own L2: the column tiles of one row chunk are given consecutive slots of
  // ONE XCD (chunk = 8 * (slot / n_ct) + xcd), so the chunk's A rows are fetched
  // into a single L2 once and shared by the blocks that run there together.
  const int n_ct = (g.N + 127) / 128;
  const int64_t slot = blockIdx.x / kXcds;
  const int64_t chunk = (slot / n_ct) * kXcds + (blockIdx.x % kXcds);
  {
    int64_t t = chunk;
    for (int r = 0; r < g.R; ++r) {
      const int64_t b = g.seg[r], e = g.seg[r + 1];
      const int64_t nt = (e - b + span - 1) / span;
      if (t < nt) { rel = r; row0 = b + t * span; row_end = e; break; }
      t -= nt;
    }
  }
  if (rel < 0) return;                       // whole block: no barrier has been passed yet
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = uniform_i32(tid >> 6);
  const bool consumer = wave < 4;
  const int n0 = (int)(slot % n_ct) * 128;
  const int K = g.K, N = g.N;
  const int64_t rows_here = (row_end - row0) < span ? (row_end - row0) : span;
  const int n_tiles = (int)((rows_here + kBM - 1) / kBM);

  // stores (or read-add-stores) of whole 16-byte pieces: this wave's 32 columns exist, rows are aligned
  // (W too: the read-add-store loads of rows that do not exist are pointed at a 16-byte piece of W)
  const bool wide_store = KS <= 8 && !g.atomic && n0 + wave * 32 + 32 <= N && (g.ldc & 3) == 0 &&
                          ((uintptr_t)g.c & 15) == 0 && ((uintptr_t)g.w & 15) == 0 &&
                          (!EPI || !g.addend || ((g.ldd & 3) == 0 && ((uintptr_t)g.addend & 15) == 0));
  // what a stored row is added to, if anything: the addend (epilogue entry point, never together
  // with accumulation) or the row of C itself
  const float* const add_src = (EPI && g.addend) ? g.addend : g.accumulate ? g.c : nullptr;
  const int64_t add_ld = (EPI && g.addend) ? g.ldd : g.ldc;

  // ---- producer state -------------------------------------------------------------
  const int ptid = tid & 255;
  const int c4 = ptid % LPR, rsub = ptid / LPR;
  const bool k_ok = 4 * c4 < K;
  const float* A = reinterpret_cast<const float*>(g.a);
  float4 areg0[NLD], areg1[NLD];             // rows of the next two tiles, in flight
  // Row tables (source and destination row of every row of a tile; -1: no such row).
  // Given row maps (MAPPED) are fetched for ALL the block's tiles before the first tile,
  // beside the consumers' weight loads: the loads of a wave complete in order, so a map
  // load inside the tile loop would make its wave wait for the row loads issued before it
  // -- the loads that are meant to stay in flight for two more tiles.  Without maps the
  // rows are the row index itself and wave 4 fills the table of tile t+4 as it goes.
  auto maps_fill = [&](int t) {
    if (!MAPPED && wave == 4 && t < n_tiles) {
      const int64_t gr = row0 + (int64_t)t * kBM + lane;
      s_src[t % SLOTS][lane] = gr < row_end ? gr : -1;
      s_dst[t % SLOTS][lane] = gr < row_end ? gr : -1;
    }
  };
  // Loads are issued unconditionally (rows and columns that do not exist are redirected
  // to an address that does; see the staging code for what happens to them): with no branch around a
  // load the compiler counts the loads in flight exactly and waits only for the older of
  // the two register sets.
  // The staging code runs from the loaded registers alone: no table look-up (an LDS read
  // and a wait per row) between the conversions.
  auto gload = [&](float4 (&areg)[NLD], int t) {
    const int tc = t < n_tiles ? t : n_tiles - 1;
    if constexpr (MAPPED) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int64_t sidx = s_src[tc % SLOTS][i * RPI + rsub];
        areg[i] = *reinterpret_cast<const float4*>(A + (sidx >= 0 ? sidx : 0) * g.lda + (k_ok ? 4 * c4 : 0));
      }
    } else {
      // consecutive rows: one base address per tile (the same for every lane, so it lives in
      // scalar registers) and a 32-bit offset per row instead of sixteen 64-bit addresses kept
      // from tile to tile -- the widest form (K up to 256: sixteen 16-byte loads per lane and
      // set) otherwise spills inside this loop, and a reload from scratch memory waits for
      // every row load in flight before it.  (The launch sees to it that 64 * lda fits.)
      const int64_t tile_row = row0 + (int64_t)tc * kBM;
      const float* const base = A + tile_row * g.lda;
      const int64_t left = row_end - tile_row;
      const int rows_here = left < kBM ? (int)left : kBM;          // at least 1
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const int rl = i * RPI + rsub;
        const unsigned off = (unsigned)(rl < rows_here ? rl : 0) * (unsigned)g.lda + (unsigned)(k_ok ? 4 * c4 : 0);
        areg[i] = *reinterpret_cast<const float4*>(base + off);
      }
    }
  };
  // split the rows held in areg and write the parts of tile t into its LDS half
  // Rows that do not exist (past the segment's end, or skipped by a negative map entry) hold
  // whatever the redirected load returned: an output row depends on its own A row only and
  // theirs is never stored, so nothing is zeroed for them.  Only the lanes past K (K below
  // the tile's 16 * KS columns) must contribute zeros, which costs one select per row.
  auto stage = [&](const float4 (&areg)[NLD], int t) {
    uint16_t (*dst)[kBM][KP] = Ap[t & 1];
    unsigned row_max[NLD];                   // F16: largest magnitude of each row (bit pattern)
    if constexpr (F16) {
#pragma unroll
      for (int i = 0; i < NLD; ++i) {
        const unsigned m = abs_max4_bits(areg[i].x, areg[i].y, areg[i].z, areg[i].w);
        row_max[i] = k_ok ? m : 0u;
      }
#pragma unroll
      for (int i = 0; i < NLD; ++i) row_max[i] = group_max_u32<LPR>(row_max[i]);
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int row = i * RPI + rsub;
      if constexpr (F16) {
        float scale, inv;
        pow2_scales(row_max[i], scale, inv);
        // (the widest form zeroes element by element instead: with the select per row its
        // register allocation spills inside the tile loop, 4.3 -> 6.0 ms at 5 M x 256 x 256)
        const float sc = (KS == 16 || k_ok) ? scale : 0.f;
        const float v[4] = {(KS < 16 || k_ok) ? areg[i].x : 0.f, (KS < 16 || k_ok) ? areg[i].y : 0.f,
                            (KS < 16 || k_ok) ? areg[i].z : 0.f, (KS < 16 || k_ok) ? areg[i].w : 0.f};
        typedef unsigned v2u __attribute__((ext_vector_type(2)));
        unsigned h01, l01, h23, l23;
        split_f16_pair(v[0], v[1], sc, h01, l01);
        split_f16_pair(v[2], v[3], sc, h23, l23);
        const v2u part[2] = {{h01, h23}, {l01, l23}};      // [high / low parts][two packed pairs]
#pragma unroll
        for (int q = 0; q < 2; ++q) *reinterpret_cast<v2u*>(&dst[q][row][4 * c4]) = part[q];
        if (c4 == 0) s_inv[t & 1][row] = inv;
      } else {
        const float v[4] = {k_ok ? areg[i].x : 0.f, k_ok ? areg[i].y : 0.f, k_ok ? areg[i].z : 0.f,
                            k_ok ? areg[i].w : 0.f};
        v4bf part[NS];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          __bf16 parts[NS];
          split_bf16<NS>(v[j], parts);
#pragma unroll
          for (int q = 0; q < NS; ++q) part[q][j] = parts[q];
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) *reinterpret_cast<v4bf*>(&dst[q][row][4 * c4]) = part[q];
      }
    }
  };

  // ---- one barrier per tile ---------------------------------------------------------
  // Each role has its prologue inside its own branch (one barrier in each): the consumers'
  // weight registers and the producers' row registers are then never live together.
  // Iteration t, consumers: multiply tile t out of LDS half t&1, store it.
  // Iteration t, producers: write the row table of tile t+4 (when no maps were given),
  // split tile t+1 into half (t+1)&1 (the consumers finished reading it before this
  // iteration's barrier), and start the loads of tile t+3 into the registers that tile
  // t+1 just left.
  // (the two kinds of waves run separate loops with the same number of barriers, so the
  // registers of one role are not live in the other)
  if (consumer) {
    if (n0 + wave * 32 >= N) {
      // all 32 columns of this wave lie past N (N <= 96 in the last column tile): nothing to
      // multiply or store, only the barriers of the block
      __syncthreads();
      for (int t = 0; t < n_tiles; ++t) __syncthreads();
      return;
    }
    v8bf bw[NS][KS];                         // this wave's 32 columns of W[rel], split (F16: fp16 bit patterns)
    float inv_w = 1.f;                       // F16: inverse scale of this lane's column
    {
      const float* W = reinterpret_cast<const float*>(g.w) + (int64_t)rel * K * N;
      const int col = n0 + wave * 32 + (lane & 31);
      if constexpr (F16) {
        // the column's largest magnitude, then its scaled parts; eight k-steps (64 values) are
        // loaded at a time, and a column of more than that is read twice (the second time out
        // of the caches)
        constexpr int HS = KS < 8 ? KS : 8;    // k-steps per batch
        float wv[HS][8];
        auto w_load = [&](int s0) {
#pragma unroll
          for (int s = 0; s < HS; ++s) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const int k = (s0 + s) * 16 + (lane >> 5) * 8 + j;
              wv[s][j] = (k < K && col < N) ? W[(int64_t)k * N + col] : 0.f;
            }
          }
        };
        unsigned m = 0;
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += HS) {
          w_load(s0);
#pragma unroll
          for (int s = 0; s < HS; ++s) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const unsigned b = __float_as_uint(wv[s][j]) & 0x7fffffffu;
              m = b > m ? b : m;
            }
          }
        }
        // the other half of the column's k range sits in lane ^ 32
        const unsigned o = (unsigned)__shfl_xor((int)m, 32, CXG_WAVE);
        m = o > m ? o : m;
        float scale;
        pow2_scales(m, scale, inv_w);
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += HS) {
          if (KS > HS) w_load(s0);             // one batch: the values are still there
#pragma unroll
          for (int s = 0; s < HS; ++s) {
            v8h h0, h1;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float xs = wv[s][j] * scale;
              h0[j] = (_Float16)xs;
              h1[j] = (_Float16)(xs - (float)h0[j]);
            }
            bw[0][s0 + s] = __builtin_bit_cast(v8bf, h0);
            bw[1][s0 + s] = __builtin_bit_cast(v8bf, h1);
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int k = s * 16 + (lane >> 5) * 8 + j;
            const float w = (k < K && col < N) ? W[(int64_t)k * N + col] : 0.f;
            __bf16 parts[NS];
            split_bf16<NS>(w, parts);
#pragma unroll
            for (int q = 0; q < NS; ++q) bw[q][s][j] = parts[q];
          }
        }
      }
    }
    __syncthreads();                         // row tables visible (all of them, or those of tiles 0..3)
    // Plain stores leave through the wave's own LDS area in row order: a lane stores 16
    // bytes and an instruction covers 8 rows x 128 bytes -- a quarter of the store
    // instructions, so four times the bytes in flight for the same depth of the memory
    // queue.  The eight pieces of tile t-1 are read back and stored between the k-steps
    // of tile t, in the shadow of its MFMAs.
    constexpr int PPS = KS <= 8 ? 8 / KS : 1;   // pieces per k-step
    auto piece_read = [&](int it) -> float4 {
      return *reinterpret_cast<const float4*>(&Cw[it * 8 + (lane >> 3)][(lane & 7) * 4]);
    };
    auto piece_row = [&](int it, int t) -> int64_t { return s_dst[t % SLOTS][it * 8 + (lane >> 3)]; };
    auto old_load = [&](int64_t d) -> float4 {
      const int colq = n0 + wave * 32 + (lane & 7) * 4;
      const float* q = d >= 0 ? add_src + d * add_ld + colq : reinterpret_cast<const float*>(g.w) + colq;
      return *reinterpret_cast<const float4*>(q);
    };
    auto piece_store = [&](const float4& v, int64_t d, auto add_tag) {
      if (d < 0) return;
      float4* const p = reinterpret_cast<float4*>(g.c + d * g.ldc + n0 + wave * 32 + (lane & 7) * 4);
      if constexpr (decltype(add_tag)::value) {
        const float4 o = *reinterpret_cast<const float4*>(add_src + d * add_ld + n0 + wave * 32 + (lane & 7) * 4);
        *p = make_float4(o.x + v.x, o.y + v.y, o.z + v.z, o.w + v.w);
      } else {
        *p = v;
      }
    };
    // this lane's accumulator column and its bias
    const int col_own = n0 + wave * 32 + (lane & 31);
    const float bias_own = (EPI && g.bias && col_own < N) ? g.bias[(int64_t)rel * N + col_own] : 0.f;
    // The tile loop exists three times, chosen once per wave (WAY 0: plain stores through the
    // LDS area, 1: the same with read-add-stores, 2: from the accumulators).  The first contains
    // no load from global memory, so the compiler puts no wait for memory into it; with all
    // kinds of store in one loop it waited at the loop's end for everything in flight, stores
    // included, because the reading paths reuse registers (7.3 M x 64 x 64 rows: 0.85 -> 0.71 ms
    // without that wait).
    auto run_tiles = [&](auto way_tag) {
    constexpr int WAY = decltype(way_tag)::value;
    constexpr bool WIDE = WAY < 2;
    constexpr std::integral_constant<bool, WAY == 1> add_tag{};
    for (int t = 0; t < n_tiles; ++t) {
      __syncthreads();
      const uint16_t (*src)[kBM][KP] = Ap[t & 1];
      const bool drain = WIDE && t > 0;
      const int tp = t > 0 ? t - 1 : 0;        // the tile whose pieces leave during this one
      float4 pv[PPS];
      int64_t pd[PPS];
      float4 po[8];                            // WAY 1: the old rows of tile t-1's pieces
      v16f acc[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;
      // operands of k-step s+1 are read while step s multiplies (two register sets)
      v8bf ap[2][2][NS];
      auto read_ap = [&](int s) {
        const int k = s * 16 + (lane >> 5) * 8;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int q = 0; q < NS; ++q)
            ap[s & 1][mt][q] = *reinterpret_cast<const v8bf*>(&src[q][mt * 32 + (lane & 31)][k]);
      };
      read_ap(0);
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        if (s + 1 < KS) read_ap(s + 1);
        if constexpr (WAY == 1) {
          // read-add-stores: the old rows of the eight pieces of tile t-1 are requested here,
          // at the start of tile t, and added and stored after its last k-step (below)
          if (s == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) po[i] = old_load(piece_row(i, tp));
          }
        } else if (drain) {
          if (s > 0) {
#pragma unroll
            for (int u = 0; u < PPS; ++u) piece_store(pv[u], pd[u], add_tag);
          }
#pragma unroll
          for (int u = 0; u < PPS; ++u) {
            pv[u] = piece_read(s * PPS + u);
            pd[u] = piece_row(s * PPS + u, t - 1);
          }
        }
        // the two accumulators alternate, so consecutive MFMAs never depend on each other
        // (k-steps past K multiply zeros: a test of K around them was measured and costs more
        // than it saves, 1.49 -> 1.91 ms at K = 128 -- it breaks the schedule of the loop)
#pragma unroll
        for (int order = NS - 1; order >= 0; --order)
#pragma unroll
          for (int i = 0; i <= order; ++i)
#pragma unroll
            for (int mt = 0; mt < 2; ++mt) {
              if constexpr (F16)
                acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, ap[s & 1][mt][i]),
                                                                 __builtin_bit_cast(v8h, bw[order - i][s]), acc[mt], 0, 0, 0);
              else
                acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ap[s & 1][mt][i], bw[order - i][s], acc[mt], 0, 0, 0);
            }
      }
      if constexpr (F16) {
        // undo the scales: accumulator element i of tile half mt is row
        // mt*32 + (i>>2)*8 + (lane>>5)*4 + (i&3), this lane's column
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float4 ri = *reinterpret_cast<const float4*>(&s_inv[t & 1][mt * 32 + q * 8 + (lane >> 5) * 4]);
            acc[mt][q * 4 + 0] *= ri.x * inv_w;
            acc[mt][q * 4 + 1] *= ri.y * inv_w;
            acc[mt][q * 4 + 2] *= ri.z * inv_w;
            acc[mt][q * 4 + 3] *= ri.w * inv_w;
          }
      }
      if constexpr (WAY == 1) {
        // Loads and stores of a wave share one in-order counter, and a store may be acknowledged
        // before an older load returns: a load that is waited for after a store can only be
        // waited for together with everything before it.  So all eight sums are formed first
        // (one wait, for loads that have had the whole tile to return) and the eight stores
        // follow with no wait between them.  The loads carry no condition (rows that do not
        // exist read a weight row instead), so the compiler counts them exactly.  (One
        // read-add-store per piece in turn, between the k-steps, made every piece a trip to
        // memory: 7.3 M x 128 x 128 rows 3.08 ms.)
        __builtin_amdgcn_sched_barrier(0);     // the sums stay behind the last k-step
        if (drain) {
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float4 v = piece_read(i);
            po[i] = make_float4(po[i].x + v.x, po[i].y + v.y, po[i].z + v.z, po[i].w + v.w);
            // (an opaque use: otherwise each sum is moved down into the branch around its store)
            asm volatile("" : "+v"(po[i].x), "+v"(po[i].y), "+v"(po[i].z), "+v"(po[i].w));
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) piece_store(po[i], piece_row(i, tp), std::false_type{});
        }
      } else if (drain) {
#pragma unroll
        for (int u = 0; u < PPS; ++u) piece_store(pv[u], pd[u], add_tag);
      }
      if (EPI && g.bias) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[mt][i] += bias_own;
      }
      if constexpr (WIDE) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            Cw[mt * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3)][lane & 31] = acc[mt][i];
      } else {
        store_tile<128, 2, EPI, 4>(g, acc, s_dst[t % SLOTS], 0, wave, lane, n0);
      }
    }
    if constexpr (WIDE) {
#pragma unroll
      for (int it = 0; it < 8; ++it) piece_store(piece_read(it), piece_row(it, n_tiles - 1), add_tag);
    }
    };
    if constexpr (KS <= 8) {
      if (wide_store && !add_src) run_tiles(std::integral_constant<int, 0>{});
      else if (wide_store) run_tiles(std::integral_constant<int, 1>{});
      else run_tiles(std::integral_constant<int, 2>{});
    } else {
      run_tiles(std::integral_constant<int, 2>{});
    }
  } else {
    if (MAPPED) {
      int64_t* const flat_src = &s_src[0][0];
      int64_t* const flat_dst = &s_dst[0][0];
      for (int i = ptid; i < n_tiles * kBM; i += 256) {          // n_tiles <= kMappedTiles (the launch sees to it)
        const int64_t gr = row0 + i;
        int64_t sidx = -1, didx = -1;
        if (gr < row_end) {
          sidx = g.src ? g.src[gr] : gr;
          didx = g.dst ? g.dst[gr] : gr;
          if (sidx < 0 || didx < 0) sidx = didx = -1;           // a negative entry in either map drops the row
        }
        flat_src[i] = sidx;
        flat_dst[i] = didx;
      }
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) maps_fill(t);
    }
    __syncthreads();                         // row tables visible
    gload(areg0, 0);
    gload(areg1, 1);
    stage(areg0, 0);
    gload(areg0, 2);
    // Two iterations per trip, so that each register set keeps a fixed role.  The loop is
    // left with `return`, never through a path that rejoins the loop head with the two
    // register sets in the other order: the compiler, which counts the loads in flight
    // statically, would then wait for every load at the head.  (Rows of four tiles in
    // flight instead of two were measured: slower, 1.81 against 1.75 ms on 7.3 M rows.)
    for (int t = 0;; t += 2) {
      if (t >= n_tiles) return;
      __syncthreads();
      maps_fill(t + 4);
      stage(areg1, t + 1);
      gload(areg1, t + 3);
      if (t + 1 >= n_tiles) return;
      __syncthreads();
      maps_fill(t + 5);
      stage(areg0, t + 2);
      gload(areg0, t + 4);
    }
  }
}

// ----------------------------------------------------------------------------
// bf16 operands, K <= 128: the same block structure as the split kernel
// ----------------------------------------------------------------------------
// A block owns up to G consecutive 64-row tiles of one relation and keeps the
// relation's W^T slab (its 32 columns per wave) in registers in B-operand layout
// -- one 16-byte load per k-step straight from W^T [R, N, K]; A rows are fetched
// as 16-byte-per-lane segments (8 bf16) and go to LDS unchanged; the loads of the
// next two tiles are in flight while the current one is multiplied.
// AF32: A and W ([R, K, N]) are fp32 in memory and rounded to bf16 (nearest even) on their way
// into the LDS and the registers -- the same result as rounding them beforehand, without the
// conversion passes and the bf16 copies.
// CBF16: the rows of C are bf16 (a compile-time choice: with the fp32 store modes -- plain,
// read-add-store, atomic -- compiled into the same kernel it needed 188 registers, two waves per
// SIMD, for a kernel whose waves each load, multiply and store in turn).
template <int KS, bool AF32, bool CBF16>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(AF32 ? 2 : 3)))
void typed_gemm_bf16_resident_kernel(GemmArgs g, int G) {
  constexpr int KP = KS * 16 + 8;          // padded LDS row (bf16 elements)
  constexpr int LPR = KS * 2;              // lanes per A row, 8 bf16 each
  constexpr int RPI = kThreads / LPR;      // rows per load instruction
  constexpr int NLD = kBM / RPI;           // load instructions per tile
  __shared__ __attribute__((aligned(16))) uint16_t Ap[kBM][KP];
  __shared__ __attribute__((aligned(16))) int64_t s_src[3][kBM], s_dst[3][kBM];
  __shared__ __attribute__((aligned(16))) uint16_t Cs[kThreads / 64][CBF16 ? 32 * kCsPitch : 8];   // bf16 rows of C on their way out
  const int64_t span = (int64_t)kBM * G;
  int rel = -1;
  int64_t row0 = 0, row_end = 0;
  const int n_ct = (g.N + 127) / 128;
  const int64_t slot = blockIdx.x / kXcds;
  const int64_t chunk = (slot / n_ct) * kXcds + (blockIdx.x % kXcds);   // see typed_gemm_split_kernel
  {
    int64_t t = chunk;
    for (int r = 0; r < g.R; ++r) {
      const int64_t b = g.seg[r], e = g.seg[r + 1];
      const int64_t nt = (e - b + span - 1) / span;
      if (t < nt) { rel = r; row0 = b + t * span; row_end = e; break; }
      t -= nt;
    }
  }
  if (rel < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = (int)(slot % n_ct) * 128;
  const int K = g.K, N = g.N;
  const int64_t rows_here = (row_end - row0) < span ? (row_end - row0) : span;
  const int n_tiles = (int)((rows_here + kBM - 1) / kBM);

  v8bf bw[KS];
  if constexpr (AF32) {
    const float* W = reinterpret_cast<const float*>(g.w) + (int64_t)rel * K * N;
    const int col = n0 + wave * 32 + (lane & 31);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = s * 16 + (lane >> 5) * 8 + j;
        bw[s][j] = (__bf16)((k < K && col < N) ? W[(int64_t)k * N + col] : 0.f);
      }
    }
  } else {
    const uint16_t* Wt = reinterpret_cast<const uint16_t*>(g.w) + (int64_t)rel * N * K;
    const int col = n0 + wave * 32 + (lane & 31);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k = s * 16 + (lane >> 5) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (col < N && k < K) v = *reinterpret_cast<const uint4*>(Wt + (int64_t)col * K + k);
      bw[s] = *reinterpret_cast<const v8bf*>(&v);
    }
  }

  const int c8 = tid % LPR, rsub = tid / LPR;
  const bool k_ok = 8 * c8 < K;
  // bf16 rows of C leave as 16-byte pieces when this wave's 32 columns exist and the rows are aligned
  const bool staged_c = CBF16 && n0 + wave * 32 + 32 <= N && (g.ldc & 7) == 0 && ((uintptr_t)g.c & 15) == 0;
  const uint16_t* A = reinterpret_cast<const uint16_t*>(g.a);
  const float* Af = reinterpret_cast<const float*>(g.a);
  constexpr int NREG = AF32 ? 2 * NLD : NLD;     // 16-byte registers per set: a row segment is 8 values
  auto load_maps = [&](int t) {
    if (tid < kBM && t < n_tiles) {
      const int64_t gr = row0 + (int64_t)t * kBM + tid;
      int64_t sidx = -1, didx = -1;
      if (gr < row_end) {
        sidx = g.src ? g.src[gr] : gr;
        didx = g.dst ? g.dst[gr] : gr;
        if (sidx < 0 || didx < 0) { sidx = -1; didx = -1; }
      }
      s_src[t % 3][tid] = sidx;
      s_dst[t % 3][tid] = didx;
    }
  };
  auto gload = [&](uint4 (&areg)[NREG], int t) {
    if (t >= n_tiles) return;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int64_t sidx = s_src[t % 3][i * RPI + rsub];
      const bool ok = sidx >= 0 && k_ok;
      if constexpr (AF32) {
        const uint4* p = reinterpret_cast<const uint4*>(Af + sidx * g.lda + 8 * c8);
        areg[2 * i] = ok ? p[0] : make_uint4(0u, 0u, 0u, 0u);
        areg[2 * i + 1] = ok ? p[1] : make_uint4(0u, 0u, 0u, 0u);
      } else {
        areg[i] = ok ? *reinterpret_cast<const uint4*>(A + sidx * g.lda + 8 * c8) : make_uint4(0u, 0u, 0u, 0u);
      }
    }
  };
  auto tile_step = [&](uint4 (&areg)[NREG], int t) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      if constexpr (AF32) {
        const uint4 lo = areg[2 * i], hi = areg[2 * i + 1];
        const float f[8] = {__uint_as_float(lo.x), __uint_as_float(lo.y), __uint_as_float(lo.z), __uint_as_float(lo.w),
                            __uint_as_float(hi.x), __uint_as_float(hi.y), __uint_as_float(hi.z), __uint_as_float(hi.w)};
        v8bf r;
#pragma unroll
        for (int j = 0; j < 8; ++j) r[j] = (__bf16)f[j];
        *reinterpret_cast<v8bf*>(&Ap[i * RPI + rsub][8 * c8]) = r;
      } else {
        *reinterpret_cast<uint4*>(&Ap[i * RPI + rsub][8 * c8]) = areg[i];
      }
    }
    load_maps(t + 2);
    __syncthreads();
    gload(areg, t + 2);
    v16f acc[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][i] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const v8bf a = *reinterpret_cast<const v8bf*>(&Ap[mt * 32 + (lane & 31)][s * 16 + (lane >> 5) * 8]);
        acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bw[s], acc[mt], 0, 0, 0);
      }
    }
    if constexpr (CBF16) {
      if (staged_c) store_tile_bf16_staged<2>(g, acc, s_dst[t % 3], wave, lane, n0, Cs[wave]);
      else store_tile_bf16<2>(g, acc, s_dst[t % 3], wave, lane, n0);
    } else {
      store_tile<128, 2>(g, acc, s_dst[t % 3], 0, wave, lane, n0);
    }
    __syncthreads();
  };
  uint4 areg0[NREG], areg1[NREG];
  load_maps(0);
  load_maps(1);
  __syncthreads();
  gload(areg0, 0);
  gload(areg1, 1);
  for (int t = 0; t < n_tiles; t += 2) {
    tile_step(areg0, t);
    if (t + 1 < n_tiles) tile_step(areg1, t + 1);
  }
}

// Dynamic LDS above the default 64 KB limit has to be enabled per kernel (once per device).
template <typename KernelT>
hipError_t allow_lds(KernelT kernel, size_t bytes) {
  if (bytes <= 64 * 1024) return hipSuccess;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)bytes);
}

int check_args(const void* a, const void* w, float* c, const int64_t* seg, int64_t M, int K, int N,
               int R, unsigned flags) {
  CXG_REQUIRE(M >= 0 && K >= 1 && N >= 1 && R >= 1, CXG_ERR_ARG, "bad M/K/N/R");
  CXG_REQUIRE((flags & ~127u) == 0, CXG_ERR_ARG, "unknown flag");
  if (M == 0) return CXG_OK;
  CXG_REQUIRE(a && w && c && seg, CXG_ERR_ARG, "null pointer");
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

static int typed_gemm_f32_impl(const float* a, int64_t lda, const float* w, const float* bias, const float* addend,
                               int64_t ldd, float* c, int64_t ldc, const int64_t* src_idx, const int64_t* dst_idx,
                               const int64_t* seg_ptr, int64_t M, int K, int N, int R, unsigned flags, void* stream) {
  int rc = cxg::check_args(a, w, c, seg_ptr, M, K, N, R, flags);
  if (rc || M == 0) return rc;
  CXG_REQUIRE(lda >= K && ldc >= N, CXG_ERR_ARG, "row stride smaller than row");
  cxg::GemmArgs g{a, lda, w, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R,
                  (int)(flags & 1u), (int)((flags >> 1) & 1u), bias, addend, ldd, (int)((flags & CXG_GEMM_OUT_BF16) != 0)};
  const bool epilogue = bias || addend;
  if (g.c_bf16) {
    CXG_REQUIRE((flags & CXG_GEMM_ROUND_BF16) && !epilogue && !(flags & 3u) && K <= 128 && (K & 7) == 0 && (lda & 7) == 0 &&
                    ((uintptr_t)a & 15) == 0 && (N & 1) == 0 && (ldc & 1) == 0 && ((uintptr_t)c & 3) == 0,
                CXG_ERR_UNSUPPORTED,
                "bf16 rows of C: with CXG_GEMM_ROUND_BF16 (K <= 128, K and lda multiples of 8), even N and ldc, plain stores");
  }
  CXG_REQUIRE(!epilogue || ((flags & CXG_GEMM_SPLIT_F16X3) && !src_idx && !dst_idx), CXG_ERR_UNSUPPORTED,
              "bias / addend are taken by the fp16 split form without row maps");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (!epilogue && (flags & CXG_GEMM_ROUND_BF16) && K <= 128 && (K & 7) == 0 && (lda & 7) == 0 && ((uintptr_t)a & 15) == 0) {
    int G = (int)(M * cxg::ceil_div(N, 128) / ((int64_t)cxg::kBM * 4096));
    G = G < 1 ? 1 : (G > 32 ? 32 : G);
    const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kBM * G) + R, cxg::kXcds) * cxg::kXcds;
    const int64_t n_blocks = n_chunks * cxg::ceil_div(N, 128);
    CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
    const dim3 grid((unsigned)n_blocks), block(cxg::kThreads);
#define CXG_RESIDENT(KSV)                                                                                     \
  do {                                                                                                        \
    if (g.c_bf16) hipLaunchKernelGGL((cxg::typed_gemm_bf16_resident_kernel<KSV, true, true>), grid, block, 0, st, g, G); \
    else hipLaunchKernelGGL((cxg::typed_gemm_bf16_resident_kernel<KSV, true, false>), grid, block, 0, st, g, G);         \
  } while (0)
    if (K <= 32) CXG_RESIDENT(2);
    else if (K <= 64) CXG_RESIDENT(4);
    else CXG_RESIDENT(8);
#undef CXG_RESIDENT
    CXG_LAUNCH_CHECK("typed_gemm_bf16_resident_kernel");
    return CXG_OK;
  }
  // Two fp16 parts of a 256-wide tile still fit the LDS: K up to 256 takes the fp16 form when the
  // 256 x 128 tile is mostly used (measured against the fp32 instructions at 7.3 M rows: K = 256,
  // N = 256 10.6 -> 5.8 ms, N = 128 5.3 -> 3.3 ms; K = 160, N = 64 2.0 -> 2.5 ms).
  const bool wide_k = (flags & CXG_GEMM_SPLIT_F16X3) && K > 128 && K <= 256 && K >= 176 && N >= 96;
  if ((flags & (CXG_GEMM_SPLIT_BF16X6 | CXG_GEMM_SPLIT_BF16X3 | CXG_GEMM_SPLIT_F16X3)) && (K <= 128 || wide_k) && (K & 3) == 0 &&
      (lda & 3) == 0 && lda < ((int64_t)1 << 24) && ((uintptr_t)a & 15) == 0) {
    // 64*G rows per block, up to 32 tiles (16 with row maps, which the block keeps in LDS).  A
    // CU runs one block at a time and a block first loads and splits its weight slab, so few
    // large blocks beat many small ones: the number of rounds of one block per CU that the
    // largest blocks would need, then the block size that fills those rounds evenly.
    const bool mapped = src_idx || dst_idx;
    const int g_max = mapped ? cxg::kMappedTiles : 32;
    const int64_t tiles = cxg::ceil_div(M, cxg::kBM) * cxg::ceil_div(N, 128);
    const int64_t rounds = cxg::ceil_div(tiles, (int64_t)256 * g_max);
    int G = (int)cxg::ceil_div(tiles, 256 * (rounds < 1 ? 1 : rounds));
    G = G < 1 ? 1 : (G > g_max ? g_max : G);
    const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kBM * G) + R, cxg::kXcds) * cxg::kXcds;
    const int64_t n_blocks = n_chunks * cxg::ceil_div(N, 128);
    CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
    const dim3 grid((unsigned)n_blocks);
#define CXG_SPLIT_LAUNCH_E(KS, NSV, MAP, HALF, EPI)                                            \
  do {                                                                                         \
    CXG_HIP_CHECK(cxg::allow_lds(cxg::typed_gemm_split_kernel<KS, NSV, MAP, HALF, EPI>, lds)); \
    hipLaunchKernelGGL((cxg::typed_gemm_split_kernel<KS, NSV, MAP, HALF, EPI>), grid, dim3(cxg::kSplitThreads), lds, \
                       st, g, G);                                                              \
  } while (0)
#define CXG_SPLIT_LAUNCH(KS, NSV, MAP, HALF) CXG_SPLIT_LAUNCH_E(KS, NSV, MAP, HALF, false)
#define CXG_SPLIT(KS)                                                                          \
  do {                                                                                         \
    const bool half = (flags & CXG_GEMM_SPLIT_F16X3) != 0;                                     \
    const int ns = (half || (flags & CXG_GEMM_SPLIT_BF16X3)) ? 2 : 3;                          \
    const size_t lds = (size_t)2 * ns * cxg::kBM * (KS * 16 + 8) * sizeof(uint16_t) +          \
                       (size_t)2 * (mapped ? cxg::kMappedTiles : cxg::kMapSlots) * cxg::kBM * sizeof(int64_t) + \
                       (KS <= 8 ? (size_t)4 * cxg::kBM * cxg::kCP * sizeof(float) : 0) +       \
                       (size_t)2 * cxg::kBM * sizeof(float);                                   \
    if (epilogue) CXG_SPLIT_LAUNCH_E(KS, 2, false, true, true);                                \
    else if (half && mapped) CXG_SPLIT_LAUNCH(KS, 2, true, true);                              \
    else if (half) CXG_SPLIT_LAUNCH(KS, 2, false, true);                                       \
    else if (ns == 2 && mapped) CXG_SPLIT_LAUNCH(KS, 2, true, false);                          \
    else if (ns == 2) CXG_SPLIT_LAUNCH(KS, 2, false, false);                                   \
    else if (mapped) CXG_SPLIT_LAUNCH(KS, 3, true, false);                                     \
    else CXG_SPLIT_LAUNCH(KS, 3, false, false);                                                \
  } while (0)
    if (K <= 32) CXG_SPLIT(2);
    else if (K <= 64) CXG_SPLIT(4);
    else if (K <= 128) CXG_SPLIT(8);
    else {                                   // 128 < K <= 256: the fp16 form only
      const size_t lds = (size_t)2 * 2 * cxg::kBM * (16 * 16 + 8) * sizeof(uint16_t) +
                         (size_t)2 * (mapped ? cxg::kMappedTiles : cxg::kMapSlots) * cxg::kBM * sizeof(int64_t) +
                         (size_t)2 * cxg::kBM * sizeof(float);
      if (epilogue) CXG_SPLIT_LAUNCH_E(16, 2, false, true, true);
      else if (mapped) CXG_SPLIT_LAUNCH(16, 2, true, true);
      else CXG_SPLIT_LAUNCH(16, 2, false, true);
    }
#undef CXG_SPLIT_LAUNCH
#undef CXG_SPLIT_LAUNCH_E
#undef CXG_SPLIT
    CXG_LAUNCH_CHECK("typed_gemm_split_kernel");
    return CXG_OK;
  }
  CXG_REQUIRE(!epilogue, CXG_ERR_UNSUPPORTED,
              "bias / addend need a split form and its shapes (K <= 128, or 176 <= K <= 256 with N >= 96 for the fp16 form)");
  const unsigned tiles = (unsigned)(cxg::ceil_div(M, cxg::kBM) + R);
  if (N > 64) {
    hipLaunchKernelGGL(cxg::typed_gemm_f32_kernel<128>, dim3(tiles, (unsigned)cxg::ceil_div(N, 128)),
                       dim3(cxg::kThreads), 0, st, g);
  } else {
    hipLaunchKernelGGL(cxg::typed_gemm_f32_kernel<64>, dim3(tiles, 1), dim3(cxg::kThreads), 0, st, g);
  }
  CXG_LAUNCH_CHECK("typed_gemm_f32_kernel");
  return CXG_OK;
}

int cxg_typed_gemm_f32(const float* a, int64_t lda, const float* w, float* c, int64_t ldc,
                       const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                       int64_t M, int K, int N, int R, unsigned flags, void* stream) {
  return typed_gemm_f32_impl(a, lda, w, nullptr, nullptr, 0, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R, flags,
                             stream);
}

int cxg_typed_gemm_epilogue_f32(const float* a, int64_t lda, const float* w, const float* bias, const float* addend,
                                int64_t ldd, float* c, int64_t ldc, const int64_t* src_idx, const int64_t* dst_idx,
                                const int64_t* seg_ptr, int64_t M, int K, int N, int R, unsigned flags, void* stream) {
  CXG_REQUIRE(!(flags & (CXG_GEMM_ATOMIC | CXG_GEMM_ACCUMULATE)), CXG_ERR_ARG,
              "bias / addend do not go with accumulation into C (pass C as the addend instead)");
  CXG_REQUIRE(!addend || ldd >= N, CXG_ERR_ARG, "addend row stride smaller than row");
  return typed_gemm_f32_impl(a, lda, w, bias, addend, ldd, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R, flags, stream);
}

int cxg_typed_gemm_bf16(const uint16_t* a, int64_t lda, const uint16_t* w_t, float* c, int64_t ldc,
                        const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                        int64_t M, int K, int N, int R, unsigned flags, void* stream) {
  int rc = cxg::check_args(a, w_t, c, seg_ptr, M, K, N, R, flags);
  if (rc || M == 0) return rc;
  CXG_REQUIRE(lda >= K && ldc >= N, CXG_ERR_ARG, "row stride smaller than row");
  CXG_REQUIRE(K % 8 == 0 && lda % 8 == 0, CXG_ERR_UNSUPPORTED, "bf16 path needs K and lda multiples of 8");
  CXG_REQUIRE(((uintptr_t)a & 15) == 0 && ((uintptr_t)w_t & 15) == 0, CXG_ERR_ARG,
              "bf16 operands must be 16-byte aligned");
  cxg::GemmArgs g{a, lda, w_t, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R,
                  (int)(flags & 1u), (int)((flags >> 1) & 1u), nullptr, nullptr, 0, (int)((flags & CXG_GEMM_OUT_BF16) != 0)};
  if (g.c_bf16) {
    CXG_REQUIRE(K <= 128 && !(flags & 3u) && (N & 1) == 0 && (ldc & 1) == 0 && ((uintptr_t)c & 3) == 0, CXG_ERR_UNSUPPORTED,
                "bf16 rows of C: K <= 128, even N and ldc, plain stores");
  }
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (K <= 128) {
    int G = (int)(M * cxg::ceil_div(N, 128) / ((int64_t)cxg::kBM * 4096));
    G = G < 1 ? 1 : (G > 32 ? 32 : G);
    const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kBM * G) + R, cxg::kXcds) * cxg::kXcds;
    const int64_t n_blocks = n_chunks * cxg::ceil_div(N, 128);
    CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
    const dim3 grid((unsigned)n_blocks), block(cxg::kThreads);
#define CXG_RESIDENT(KSV)                                                                                     \
  do {                                                                                                        \
    if (g.c_bf16) hipLaunchKernelGGL((cxg::typed_gemm_bf16_resident_kernel<KSV, false, true>), grid, block, 0, st, g, G); \
    else hipLaunchKernelGGL((cxg::typed_gemm_bf16_resident_kernel<KSV, false, false>), grid, block, 0, st, g, G);         \
  } while (0)
    if (K <= 32) CXG_RESIDENT(2);
    else if (K <= 64) CXG_RESIDENT(4);
    else CXG_RESIDENT(8);
#undef CXG_RESIDENT
    CXG_LAUNCH_CHECK("typed_gemm_bf16_resident_kernel");
    return CXG_OK;
  }
  const unsigned tiles = (unsigned)(cxg::ceil_div(M, cxg::kBM) + R);
  if (N > 64) {
    hipLaunchKernelGGL(cxg::typed_gemm_bf16_kernel<128>, dim3(tiles, (unsigned)cxg::ceil_div(N, 128)),
                       dim3(cxg::kThreads), 0, st, g);
  } else {
    hipLaunchKernelGGL(cxg::typed_gemm_bf16_kernel<64>, dim3(tiles, 1), dim3(cxg::kThreads), 0, st, g);
  }
  CXG_LAUNCH_CHECK("typed_gemm_bf16_kernel");
  return CXG_OK;
}

}  // extern "C"
