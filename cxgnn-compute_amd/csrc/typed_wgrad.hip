// Weight gradient of the typed GEMM on the gfx950 matrix cores:
//
//   gW[r] (K x N)  =  sum over the rows i of segment r of  A[src(i), :]^T  (x)  G[dst(i), :]
//
// i.e. a GEMM whose reduction runs over the (gathered) rows.  fp32 operands are
// split into NS bf16 parts and multiplied as partial products on
// v_mfma_f32_32x32x16_bf16 exactly as in the forward kernel (NS = 3: six products,
// fp32-accurate; NS = 2: three products).
//
// The MFMA wants eight consecutive reduction indices per lane, and the reduction
// index is the row index of both operands in memory, so both tiles are transposed
// on their way into LDS: a thread fetches one float4 from each of 4 consecutive
// rows (coalesced along the row), and writes, for each of its 4 columns, the 4
// row-consecutive bf16 values as one 8-byte LDS store into [column][row] order.
//
// Split over the rows: a block owns `rows_per_chunk` rows of one relation and one
// 128-column tile of G, keeps the 128 x 128 partial in registers (wave w: output
// rows 32w .. 32w+31) and writes it to a partial buffer; a second kernel adds the
// partials of each relation in chunk order -- no atomics, deterministic.
//
// Replaces the weight-gradient half of TypedLinearE2EOP.backward /
// TypedLinearS2DMMAggrOP.backward (cxgnncomp/typed_linear.py:114-137,205-221),
// which the reference computes with one torch.mm per relation.
#include "cxg_common.hpp"

namespace cxg {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kXcds = 8;                 // accelerator dies of an MI355X, one L2 each
constexpr int kMT = 32;                  // rows per step
constexpr int kMP = kMT + 8;             // padded row extent in LDS (bf16 elements): 80-byte pitch

struct WgradArgs {
  const float* a;
  int64_t lda;
  const float* g;
  int64_t ldg;
  const int64_t* src;
  const int64_t* dst;
  const int64_t* seg;
  float* partial;
  int64_t M;
  int K, N, R;
  int64_t rows_per_chunk;
};

template <int NS>
__device__ __forceinline__ void split_parts(float x, __bf16 (&p)[NS]) {
#pragma unroll
  for (int i = 0; i < NS; ++i) {
    p[i] = (__bf16)x;
    x -= (float)p[i];
  }
}

// Chunk number -> (relation, first row, end of the relation's rows); block-uniform.
__device__ __forceinline__ bool locate_chunk(const int64_t* __restrict__ seg, int R, int64_t span,
                                             int64_t chunk, int& rel, int64_t& row0, int64_t& row_end) {
  int64_t t = chunk;
  for (int r = 0; r < R; ++r) {
    const int64_t b = seg[r], e = seg[r + 1];
    const int64_t nt = (e - b + span - 1) / span;
    if (t < nt) { rel = r; row0 = b + t * span; row_end = e; return true; }
    t -= nt;
  }
  return false;
}

template <int NS>
__global__ __launch_bounds__(kThreads) void typed_wgrad_split_kernel(WgradArgs g) {
  __shared__ __attribute__((aligned(16))) uint16_t At[NS][128][kMP];   // [part][k][row]
  __shared__ __attribute__((aligned(16))) uint16_t Gt[NS][128][kMP];   // [part][n][row]
  __shared__ int64_t s_src[3][kMT], s_dst[3][kMT];
  // The column tiles of one row chunk get consecutive slots of one XCD (blocks go to
  // the 8 XCDs round-robin by index), so the chunk's A rows are fetched into one L2.
  const int n_ct = (g.N + 127) / 128;
  const int64_t slot = blockIdx.x / kXcds;
  const int64_t chunk = (slot / n_ct) * kXcds + (blockIdx.x % kXcds);
  const int n0 = (int)(slot % n_ct) * 128;
  int rel = 0;
  int64_t row0 = 0, row_end = 0;
  const bool have = locate_chunk(g.seg, g.R, g.rows_per_chunk, chunk, rel, row0, row_end);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = g.K, N = g.N;
  float* const part = g.partial + ((size_t)chunk * K) * (size_t)N;
  v16f acc[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nb][i] = 0.f;

  if (have) {
    const int64_t rows_here = (row_end - row0) < g.rows_per_chunk ? (row_end - row0) : g.rows_per_chunk;
    const int n_tiles = (int)((rows_here + kMT - 1) / kMT);
    // float4 column and group of 4 rows of this thread: 8 lanes run along a row (128
    // contiguous bytes per global load), the other lane bits select the row group, so
    // the transposed 8-byte LDS stores of a wave spread over the banks (2-way conflicts
    // at most with the 80-byte pitch) instead of piling onto four of them.
    const int c4 = wave * 8 + (lane & 7), mg = lane >> 3;
    const bool ka_ok = 4 * c4 < K;
    const bool ng_ok = n0 + 4 * c4 < N;               // N % 4 == 0 is required
    auto load_maps = [&](int t) {
      if (tid < kMT && t < n_tiles) {
        const int64_t gr = row0 + (int64_t)t * kMT + tid;
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
    // Loads are issued unconditionally: rows and columns that do not exist are redirected
    // to an address that does and zeroed when the tile is staged (a select between a
    // loaded vector and a zero vector made the compiler route the load through scratch).
    auto gload = [&](float4 (&ar)[4], float4 (&gr4)[4], int t) {
      const int tc = t < n_tiles ? t : n_tiles - 1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t sidx = s_src[tc % 3][mg * 4 + i], didx = s_dst[tc % 3][mg * 4 + i];
        ar[i] = *reinterpret_cast<const float4*>(g.a + (sidx >= 0 ? sidx : 0) * g.lda + (ka_ok ? 4 * c4 : 0));
        gr4[i] = *reinterpret_cast<const float4*>(g.g + (didx >= 0 ? didx : 0) * g.ldg + (ng_ok ? n0 + 4 * c4 : 0));
      }
    };
    // registers (4 rows x 4 columns) -> LDS [column][4 consecutive rows], split into parts
    auto stage = [&](const float4 (&r4)[4], uint16_t (&dst)[NS][128][kMP], const int64_t* rows, bool col_ok) {
      float v[4][4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool live = col_ok && rows[mg * 4 + i] >= 0;
        v[i][0] = live ? r4[i].x : 0.f;
        v[i][1] = live ? r4[i].y : 0.f;
        v[i][2] = live ? r4[i].z : 0.f;
        v[i][3] = live ? r4[i].w : 0.f;
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        v4bf out[NS];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          __bf16 p[NS];
          split_parts<NS>(v[i][c], p);
#pragma unroll
          for (int q = 0; q < NS; ++q) out[q][i] = p[q];
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) *reinterpret_cast<v4bf*>(&dst[q][4 * c4 + c][mg * 4]) = out[q];
      }
    };
    auto tile_step = [&](float4 (&ar)[4], float4 (&gr4)[4], int t) {
      stage(ar, At, s_src[t % 3], ka_ok);
      stage(gr4, Gt, s_dst[t % 3], ng_ok);
      load_maps(t + 2);
      __syncthreads();
      gload(ar, gr4, t + 2);
#pragma unroll
      for (int ms = 0; ms < kMT / 16; ++ms) {
        const int m = ms * 16 + (lane >> 5) * 8;
        v8bf af[NS];
#pragma unroll
        for (int q = 0; q < NS; ++q) af[q] = *reinterpret_cast<const v8bf*>(&At[q][wave * 32 + (lane & 31)][m]);
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          v8bf bf[NS];
#pragma unroll
          for (int q = 0; q < NS; ++q) bf[q] = *reinterpret_cast<const v8bf*>(&Gt[q][nb * 32 + (lane & 31)][m]);
#pragma unroll
          for (int order = NS - 1; order >= 0; --order)
#pragma unroll
            for (int i = 0; i <= order; ++i)
              acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[order - i], acc[nb], 0, 0, 0);
        }
      }
      __syncthreads();   // every wave is done with At / Gt before the next tile is staged
    };
    float4 a0[4], g0[4], a1[4], g1[4];
    load_maps(0);
    load_maps(1);
    __syncthreads();
    gload(a0, g0, 0);
    gload(a1, g1, 1);
    for (int t = 0; t < n_tiles; t += 2) {
      tile_step(a0, g0, t);
      if (t + 1 < n_tiles) tile_step(a1, g1, t + 1);
    }
  }
  // partial[chunk][k][n] (zeros for chunk numbers past the last relation)
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int col = n0 + nb * 32 + (lane & 31);
    if (col >= N) continue;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int k = wave * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
      if (k < K) part[(size_t)k * N + col] = acc[nb][i];
    }
  }
}

// gw[r][k][n] = sum of the partials of relation r's chunks, in a fixed order: the chunks
// are cut into kReduceSlices contiguous runs, each run is summed by one thread (four
// interleaved chains, so the loads overlap) and the runs are added in run order.
constexpr int kReduceSlices = 4;

__global__ __launch_bounds__(64 * kReduceSlices) void wgrad_reduce_kernel(
    const int64_t* __restrict__ seg, int R, int64_t rows_per_chunk, const float* __restrict__ partial,
    float* __restrict__ gw, int64_t kn) {
  __shared__ float s_run[kReduceSlices][64];
  const int el = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int64_t e = (int64_t)blockIdx.x * 64 + el;
  const int r = blockIdx.y;
  int64_t first = 0;
  for (int q = 0; q < r; ++q) first += (seg[q + 1] - seg[q] + rows_per_chunk - 1) / rows_per_chunk;
  const int64_t cnt = (seg[r + 1] - seg[r] + rows_per_chunk - 1) / rows_per_chunk;
  const int64_t per = (cnt + kReduceSlices - 1) / kReduceSlices;
  const int64_t c0 = sl * per, c1 = (c0 + per) < cnt ? (c0 + per) : cnt;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
  if (e < kn) {
    const float* p = partial + (size_t)first * kn + e;
    int64_t c = c0;
    for (; c + 4 <= c1; c += 4) {
      a0 += p[(size_t)(c + 0) * kn];
      a1 += p[(size_t)(c + 1) * kn];
      a2 += p[(size_t)(c + 2) * kn];
      a3 += p[(size_t)(c + 3) * kn];
    }
    for (; c < c1; ++c) a0 += p[(size_t)c * kn];
  }
  s_run[sl][el] = (a0 + a1) + (a2 + a3);
  __syncthreads();
  if (sl == 0 && e < kn) {
    float acc = s_run[0][el];
#pragma unroll
    for (int q = 1; q < kReduceSlices; ++q) acc += s_run[q][el];
    gw[(size_t)r * kn + e] = acc;
  }
}

int64_t chunk_rows(int64_t M, int N) {
  int64_t rows = M * ceil_div(N, 128) / 4096;
  rows = (rows + kMT - 1) / kMT * kMT;
  if (rows < 8 * kMT) rows = 8 * kMT;
  if (rows > 256 * kMT) rows = 256 * kMT;
  return rows;
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_typed_gemm_wgrad_workspace_bytes(int64_t M, int K, int N, int R) {
  if (M < 0 || K < 1 || N < 1 || R < 1) return 0;
  const int64_t chunks = cxg::ceil_div(cxg::ceil_div(M, cxg::chunk_rows(M, N)) + R, cxg::kXcds) * cxg::kXcds;
  return (size_t)chunks * (size_t)K * (size_t)N * sizeof(float) + 256;
}

int cxg_typed_gemm_wgrad_f32(const float* a, int64_t lda, const float* g, int64_t ldg,
                             const int64_t* src_idx, const int64_t* dst_idx, const int64_t* seg_ptr,
                             int64_t M, int K, int N, int R, float* gw, unsigned flags, void* workspace,
                             size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(M >= 0 && K >= 1 && N >= 1 && R >= 1, CXG_ERR_ARG, "bad M/K/N/R");
  CXG_REQUIRE((flags & ~(CXG_GEMM_SPLIT_BF16X6 | CXG_GEMM_SPLIT_BF16X3)) == 0, CXG_ERR_ARG, "unknown flag");
  CXG_REQUIRE(gw && seg_ptr, CXG_ERR_ARG, "null gw/seg_ptr");
  CXG_REQUIRE(M == 0 || (a && g), CXG_ERR_ARG, "null a/g");
  CXG_REQUIRE(K <= 128 && (K & 3) == 0 && (N & 3) == 0 && (lda & 3) == 0 && (ldg & 3) == 0 &&
                  ((uintptr_t)a & 15) == 0 && ((uintptr_t)g & 15) == 0,
              CXG_ERR_UNSUPPORTED, "wgrad needs K <= 128, K, N, lda, ldg multiples of 4 and 16-byte aligned operands");
  CXG_REQUIRE(lda >= K && ldg >= N, CXG_ERR_ARG, "row stride smaller than row");
  const size_t need = cxg_typed_gemm_wgrad_workspace_bytes(M, K, N, R);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t rows = cxg::chunk_rows(M, N);
  const int64_t chunks = cxg::ceil_div(cxg::ceil_div(M, rows) + R, cxg::kXcds) * cxg::kXcds;
  const int n_ct = (int)cxg::ceil_div(N, 128);
  CXG_REQUIRE(chunks * n_ct < ((int64_t)1 << 31), CXG_ERR_UNSUPPORTED, "too many chunks for one launch");
  cxg::WgradArgs wa{a, lda, g, ldg, src_idx, dst_idx, seg_ptr, reinterpret_cast<float*>(workspace),
                    M, K, N, R, rows};
  const dim3 grid((unsigned)(chunks * n_ct)), block(cxg::kThreads);
  if (flags & CXG_GEMM_SPLIT_BF16X3) hipLaunchKernelGGL(cxg::typed_wgrad_split_kernel<2>, grid, block, 0, st, wa);
  else hipLaunchKernelGGL(cxg::typed_wgrad_split_kernel<3>, grid, block, 0, st, wa);
  CXG_LAUNCH_CHECK("typed_wgrad_split_kernel");
  const int64_t kn = (int64_t)K * N;
  hipLaunchKernelGGL(cxg::wgrad_reduce_kernel, dim3((unsigned)cxg::ceil_div(kn, 64), (unsigned)R),
                     dim3(64 * cxg::kReduceSlices), 0,
                     st, seg_ptr, R, rows, reinterpret_cast<const float*>(workspace), gw, kn);
  CXG_LAUNCH_CHECK("wgrad_reduce_kernel");
  return CXG_OK;
}

}  // extern "C"
