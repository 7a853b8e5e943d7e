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
#include "cxg_common.hpp"

namespace cxg {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

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

template <int BN, int MT>
__device__ __forceinline__ void store_tile(const GemmArgs& g, const v16f (&acc)[MT],
                                           const int64_t* s_dst, int wm, int wn, int lane, int n0) {
  const int col = n0 + wn * 32 + (lane & 31);
  if (col >= g.N) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int rl = (wm * MT + mt) * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
      const int64_t d = s_dst[rl];
      if (d < 0) continue;
      float* p = g.c + d * g.ldc + col;
      const float v = acc[mt][i];
      if (g.atomic) unsafeAtomicAdd(p, v);
      else if (g.accumulate) *p += v;
      else *p = v;
    }
  }
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
  __shared__ int64_t s_src[kBM], s_dst[kBM];
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
  __shared__ int64_t s_src[kBM], s_dst[kBM];
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
// A block owns up to G consecutive 64-row tiles of ONE relation and keeps that
// relation's weight slab in registers, already split and in MFMA operand layout
// (wave w: columns 32w..32w+31), so W is fetched once per 64*G rows.  A tiles are
// fetched as whole 16-byte-per-lane row segments, split on the way into LDS, and
// the loads of the next two tiles are in flight while the current one is multiplied.
template <int NS>
__device__ __forceinline__ void split_bf16(float x, __bf16 (&p)[NS]) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    p[i] = (__bf16)x;
    x -= (float)p[i];
  }
}

template <int KS, int NS>
__global__ __launch_bounds__(kThreads) void typed_gemm_split_kernel(GemmArgs g, int G) {
  constexpr int KP = KS * 16 + 8;          // padded LDS row (bf16 elements)
  constexpr int LPR = KS * 4;              // lanes per A row, one float4 each
  constexpr int RPI = kThreads / LPR;      // rows per load instruction
  constexpr int NLD = kBM / RPI;           // load instructions per tile
  __shared__ __attribute__((aligned(16))) uint16_t Ap[NS][kBM][KP];
  __shared__ int64_t s_src[3][kBM], s_dst[3][kBM];
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
  if (rel < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = (int)(slot % n_ct) * 128;
  const int K = g.K, N = g.N;
  const int64_t rows_here = (row_end - row0) < span ? (row_end - row0) : span;
  const int n_tiles = (int)((rows_here + kBM - 1) / kBM);

  // this wave's 32 columns of W[rel], split, in B-operand layout
  v8bf bw[NS][KS];
  {
    const float* W = reinterpret_cast<const float*>(g.w) + (int64_t)rel * K * N;
    const int col = n0 + wave * 32 + (lane & 31);
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

  const int c4 = tid % LPR, rsub = tid / LPR;
  const bool k_ok = 4 * c4 < K;
  const float* A = reinterpret_cast<const float*>(g.a);
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
  auto gload = [&](float4 (&areg)[NLD], int t) {
    if (t >= n_tiles) return;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int64_t sidx = s_src[t % 3][i * RPI + rsub];
      areg[i] = (sidx >= 0 && k_ok) ? *reinterpret_cast<const float4*>(A + sidx * g.lda + 4 * c4)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  // One tile: stage its rows (already in registers) into LDS, start the loads of
  // tile t + 2 into the same registers, multiply, store.
  auto tile_step = [&](float4 (&areg)[NLD], int t) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const float v[4] = {areg[i].x, areg[i].y, areg[i].z, areg[i].w};
      typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
      v4bf part[NS];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        __bf16 parts[NS];
        split_bf16<NS>(v[j], parts);
#pragma unroll
        for (int q = 0; q < NS; ++q) part[q][j] = parts[q];
      }
      const int row = i * RPI + rsub;
#pragma unroll
      for (int q = 0; q < NS; ++q) *reinterpret_cast<v4bf*>(&Ap[q][row][4 * c4]) = part[q];
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
        const int row = mt * 32 + (lane & 31), k = s * 16 + (lane >> 5) * 8;
        v8bf ap[NS];
#pragma unroll
        for (int q = 0; q < NS; ++q) ap[q] = *reinterpret_cast<const v8bf*>(&Ap[q][row][k]);
#pragma unroll
        for (int order = NS - 1; order >= 0; --order)
#pragma unroll
          for (int i = 0; i <= order; ++i)
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ap[i], bw[order - i][s], acc[mt], 0, 0, 0);
      }
    }
    store_tile<128, 2>(g, acc, s_dst[t % 3], 0, wave, lane, n0);
    __syncthreads();   // every wave is done with Ap before the next tile is staged
  };

  float4 areg0[NLD], areg1[NLD];
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

// ----------------------------------------------------------------------------
// bf16 operands, K <= 128: the same block structure as the split kernel
// ----------------------------------------------------------------------------
// A block owns up to G consecutive 64-row tiles of one relation and keeps the
// relation's W^T slab (its 32 columns per wave) in registers in B-operand layout
// -- one 16-byte load per k-step straight from W^T [R, N, K]; A rows are fetched
// as 16-byte-per-lane segments (8 bf16) and go to LDS unchanged; the loads of the
// next two tiles are in flight while the current one is multiplied.
template <int KS>
__global__ __launch_bounds__(kThreads) void typed_gemm_bf16_resident_kernel(GemmArgs g, int G) {
  constexpr int KP = KS * 16 + 8;          // padded LDS row (bf16 elements)
  constexpr int LPR = KS * 2;              // lanes per A row, 8 bf16 each
  constexpr int RPI = kThreads / LPR;      // rows per load instruction
  constexpr int NLD = kBM / RPI;           // load instructions per tile
  __shared__ __attribute__((aligned(16))) uint16_t Ap[kBM][KP];
  __shared__ int64_t s_src[3][kBM], s_dst[3][kBM];
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
  {
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
  const uint16_t* A = reinterpret_cast<const uint16_t*>(g.a);
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
  auto gload = [&](uint4 (&areg)[NLD], int t) {
    if (t >= n_tiles) return;
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int64_t sidx = s_src[t % 3][i * RPI + rsub];
      areg[i] = (sidx >= 0 && k_ok) ? *reinterpret_cast<const uint4*>(A + sidx * g.lda + 8 * c8)
                                    : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  auto tile_step = [&](uint4 (&areg)[NLD], int t) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) *reinterpret_cast<uint4*>(&Ap[i * RPI + rsub][8 * c8]) = areg[i];
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
    store_tile<128, 2>(g, acc, s_dst[t % 3], 0, wave, lane, n0);
    __syncthreads();
  };
  uint4 areg0[NLD], areg1[NLD];
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

int check_args(const void* a, const void* w, float* c, const int64_t* seg, int64_t M, int K, int N,
               int R, unsigned flags) {
  CXG_REQUIRE(M >= 0 && K >= 1 && N >= 1 && R >= 1, CXG_ERR_ARG, "bad M/K/N/R");
  CXG_REQUIRE((flags & ~15u) == 0, CXG_ERR_ARG, "unknown flag");
  if (M == 0) return CXG_OK;
  CXG_REQUIRE(a && w && c && seg, CXG_ERR_ARG, "null pointer");
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_typed_gemm_f32(const float* a, int64_t lda, const float* w, float* c, int64_t ldc,
                       const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                       int64_t M, int K, int N, int R, unsigned flags, void* stream) {
  int rc = cxg::check_args(a, w, c, seg_ptr, M, K, N, R, flags);
  if (rc || M == 0) return rc;
  CXG_REQUIRE(lda >= K && ldc >= N, CXG_ERR_ARG, "row stride smaller than row");
  cxg::GemmArgs g{a, lda, w, c, ldc, src_idx, dst_idx, seg_ptr, M, K, N, R,
                  (int)(flags & 1u), (int)((flags >> 1) & 1u)};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if ((flags & (CXG_GEMM_SPLIT_BF16X6 | CXG_GEMM_SPLIT_BF16X3)) && K <= 128 && (K & 3) == 0 && (lda & 3) == 0 &&
      ((uintptr_t)a & 15) == 0) {
    // 64*G rows per block: up to 32 tiles while the launch keeps a few thousand blocks
    int G = (int)(M * cxg::ceil_div(N, 128) / ((int64_t)cxg::kBM * 4096));
    G = G < 1 ? 1 : (G > 32 ? 32 : G);
    const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kBM * G) + R, cxg::kXcds) * cxg::kXcds;
    const int64_t n_blocks = n_chunks * cxg::ceil_div(N, 128);
    CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
    const dim3 grid((unsigned)n_blocks);
#define CXG_SPLIT(KS)                                                                          \
  do {                                                                                         \
    if (flags & CXG_GEMM_SPLIT_BF16X3)                                                         \
      hipLaunchKernelGGL((cxg::typed_gemm_split_kernel<KS, 2>), grid, dim3(cxg::kThreads), 0, st, g, G); \
    else                                                                                       \
      hipLaunchKernelGGL((cxg::typed_gemm_split_kernel<KS, 3>), grid, dim3(cxg::kThreads), 0, st, g, G); \
  } while (0)
    if (K <= 32) CXG_SPLIT(2);
    else if (K <= 64) CXG_SPLIT(4);
    else CXG_SPLIT(8);
#undef CXG_SPLIT
    CXG_LAUNCH_CHECK("typed_gemm_split_kernel");
    return CXG_OK;
  }
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
                  (int)(flags & 1u), (int)((flags >> 1) & 1u)};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (K <= 128) {
    int G = (int)(M * cxg::ceil_div(N, 128) / ((int64_t)cxg::kBM * 4096));
    G = G < 1 ? 1 : (G > 32 ? 32 : G);
    const int64_t n_chunks = cxg::ceil_div(cxg::ceil_div(M, (int64_t)cxg::kBM * G) + R, cxg::kXcds) * cxg::kXcds;
    const int64_t n_blocks = n_chunks * cxg::ceil_div(N, 128);
    CXG_REQUIRE(n_blocks < (int64_t)1 << 31, CXG_ERR_UNSUPPORTED, "too many tiles for one launch");
    const dim3 grid((unsigned)n_blocks), block(cxg::kThreads);
    if (K <= 32) hipLaunchKernelGGL(cxg::typed_gemm_bf16_resident_kernel<2>, grid, block, 0, st, g, G);
    else if (K <= 64) hipLaunchKernelGGL(cxg::typed_gemm_bf16_resident_kernel<4>, grid, block, 0, st, g, G);
    else hipLaunchKernelGGL(cxg::typed_gemm_bf16_resident_kernel<8>, grid, block, 0, st, g, G);
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
