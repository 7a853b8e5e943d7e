// Generalised CSR SpMM with int32 indices, the entry points the reference
// takes from dgSPARSE (GSpMM_u / GSpMM_u_e, src/cpp/include/dgsparse.h:14-131,
// src/cpp/src/dgsparse.cu:6-474):
//
//   out[r, c] = REDUCE_{e in row r} COMPUTE(val[e], b[colind[e], c])
//
// REDUCE sum / max / min / mean, COMPUTE val+b / b-val / val*b / b/val.  The
// accumulator of a non-empty row starts at the reference's init(op) (0,
// (float)INT_MIN, (float)INT_MAX, 0), empty rows give 0, mean divides by the
// row length.
//
// One wave per (row, column tile).  A lane holds V consecutive output columns (V = 4 when
// the row width allows 16-byte accesses), an edge occupies L = tile/V lanes (a power of
// two) and the wave works on 64/L edges of the row at once, four rounds unrolled; the
// row's column ids (and values) are fetched 64 at a time with one coalesced load and
// handed out by lane shuffles; the edge groups are combined with the reduction operator
// at the end of the row.  A row of more than kLongRow edges would keep one wave busy long
// after the rest of the grid has drained, so such rows are cut at the multiples of
// kLongRow in the edge array: a first kernel gives every cut piece to a wave of its own and
// leaves one partial row per piece in the workspace (a piece of kLongRow edges meets at
// most two long rows: the one holding its first edge and the one holding its last), and
// the row kernel then folds the partials of a long row in edge order, so the result does
// not depend on the schedule.  Sum and mean without edge values are served by the
// edge-span SpMM kernel instead (the host wrapper routes them there); this kernel covers
// the combinations that kernel has no carry rule for.
#include "cxg_common.hpp"

#include <climits>

namespace cxg {
namespace {

constexpr int kBlock = 256;

template <int RED>
__device__ __forceinline__ float reduce_op(float acc, float t) {
  if (RED == 1) return acc < t ? t : acc;
  if (RED == 2) return t < acc ? t : acc;
  return acc + t;
}
template <int COMP>
__device__ __forceinline__ float compute_op(float v, float f) {
  if (COMP == 0) return v + f;
  if (COMP == 1) return f - v;
  if (COMP == 2) return v * f;
  return f / v;
}

template <int V> struct GVec;
template <> struct GVec<1> { using type = float; };
template <> struct GVec<4> { using type = float4; };

template <int RED, int COMP, bool HASVAL>
__device__ __forceinline__ void accumulate(float& acc, float v, float f) {
  acc = reduce_op<RED>(acc, HASVAL ? compute_op<COMP>(v, f) : f);
}

constexpr int kRounds = 4;               // edge rounds in flight per group
constexpr int kLongRow = 512;            // rows above this many edges are cut into pieces of this size

// Edges [lb, hb) of one row folded into acc: the wave's 64/L edge groups each keep their own
// accumulator (all start from the same value), the caller combines them.
template <int RED, int COMP, bool HASVAL, int V>
__device__ __forceinline__ void fold_edges(const int32_t* __restrict__ colind,
                                           const float* __restrict__ val,
                                           const float* __restrict__ b, int feat, int lb, int hb,
                                           int lane, int L, int col, bool col_ok, float (&acc)[V]) {
  using vec_t = typename GVec<V>::type;
  const int G = CXG_WAVE / L;              // edges per round
  const int es = lane / L;
  for (int c0 = lb; c0 < hb; c0 += CXG_WAVE) {
    const int cn = hb - c0 < CXG_WAVE ? hb - c0 : CXG_WAVE;
    int my_col = 0;
    float my_val = 0.f;
    if (lane < cn) {
      my_col = colind[c0 + lane];
      if (HASVAL) my_val = val[c0 + lane];
    }
    for (int j0 = 0; j0 < cn; j0 += kRounds * G) {
      float f[kRounds][V], v[kRounds];
      bool on[kRounds];
#pragma unroll
      for (int u = 0; u < kRounds; ++u) {
        const int j = j0 + u * G + es;
        on[u] = j < cn && col_ok;
        const int64_t src = __shfl(my_col, j & 63, CXG_WAVE);
        v[u] = HASVAL ? __shfl(my_val, j & 63, CXG_WAVE) : 0.f;
        if (on[u]) {
          const vec_t t = *reinterpret_cast<const vec_t*>(b + src * feat + col);
          __builtin_memcpy(f[u], &t, sizeof(vec_t));
        }
      }
#pragma unroll
      for (int u = 0; u < kRounds; ++u)
        if (on[u])
#pragma unroll
          for (int i = 0; i < V; ++i) accumulate<RED, COMP, HASVAL>(acc[i], v[u], f[u][i]);
    }
  }
}

// the edge groups of the wave folded into every lane (all groups started from the same value)
template <int RED, int V>
__device__ __forceinline__ void combine_groups(float (&acc)[V], int L) {
  for (int m = L; m < CXG_WAVE; m <<= 1)
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = reduce_op<RED>(acc[i], __shfl_xor(acc[i], m, CXG_WAVE));
}

// last row whose first edge is at or before edge e (rows without edges are stepped over);
// the same value in every lane
__device__ __forceinline__ int row_of_edge(const int32_t* __restrict__ rowptr, int64_t n_rows, int e) {
  int lo = 0, hi = (int)n_rows;            // answer in [lo, hi): rowptr[lo] <= e < rowptr[hi]
  while (hi - lo > 1) {
    const int mid = lo + ((hi - lo) >> 1);
    if (rowptr[mid] <= e) lo = mid; else hi = mid;
  }
  return lo;
}

// One wave per (piece of kLongRow edges, column tile): the partial rows of the long rows
// that hold the piece's first edge (slot 0) and its last edge (slot 1, when that row starts
// inside the piece).
template <int RED, int COMP, bool HASVAL, int V>
__global__ __launch_bounds__(kBlock) void gspmm_long_rows_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
    const float* __restrict__ val, const float* __restrict__ b, float* __restrict__ ws,
    int64_t n_rows, int64_t n_pieces, int feat, float ini, int L) {
  using vec_t = typename GVec<V>::type;
  const int lane = lane_id();
  const int64_t piece = (int64_t)blockIdx.x * (kBlock / CXG_WAVE) + uniform_i32(threadIdx.x >> 6);
  if (piece >= n_pieces) return;
  const int first = rowptr[0], last = rowptr[n_rows];
  const int64_t a64 = piece * kLongRow, z64 = a64 + kLongRow;     // z64 may pass 2^31 in the last piece
  const int a = a64 < first ? first : (int)a64;
  const int z = z64 > last ? last : (int)z64;
  if (a >= z) return;
  const int col = (blockIdx.y * L + lane % L) * V;
  const bool col_ok = col < feat;
  const int r0 = row_of_edge(rowptr, n_rows, a), r1 = row_of_edge(rowptr, n_rows, z - 1);
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int r = k ? r1 : r0;
    if (k && r1 == r0) break;
    const int lb = rowptr[r], hb = rowptr[r + 1];
    if (hb - lb <= kLongRow) continue;
    const int slot = lb <= piece * kLongRow ? 0 : 1;     // the rule the row kernel reads by
    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = ini;
    fold_edges<RED, COMP, HASVAL, V>(colind, val, b, feat, lb > a ? lb : a, hb < z ? hb : z, lane, L, col,
                                     col_ok, acc);
    combine_groups<RED, V>(acc, L);
    if (col_ok && lane < L) {
      vec_t t;
      __builtin_memcpy(&t, acc, sizeof(vec_t));
      *reinterpret_cast<vec_t*>(ws + (piece * 2 + slot) * feat + col) = t;
    }
  }
}

template <int RED, int COMP, bool HASVAL, int V>
__global__ __launch_bounds__(kBlock) void gspmm_row_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
    const float* __restrict__ val, const float* __restrict__ b, float* __restrict__ out,
    const float* __restrict__ ws, int64_t n_rows, int feat, float ini, int L) {
  using vec_t = typename GVec<V>::type;
  const int lane = lane_id();
  const int64_t r = (int64_t)blockIdx.x * (kBlock / CXG_WAVE) + uniform_i32(threadIdx.x >> 6);
  if (r >= n_rows) return;
  const int col = (blockIdx.y * L + lane % L) * V;
  const bool col_ok = col < feat;          // feat % V == 0: a lane's V columns exist together
  const int lb = rowptr[r], hb = rowptr[r + 1];
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = hb > lb ? ini : 0.f;
  if (hb - lb <= kLongRow) {
    fold_edges<RED, COMP, HASVAL, V>(colind, val, b, feat, lb, hb, lane, L, col, col_ok, acc);
    combine_groups<RED, V>(acc, L);
  } else if (col_ok) {
    // the partial rows of the pieces this row runs through, in edge order
    for (int64_t piece = lb / kLongRow; piece <= (hb - 1) / kLongRow; ++piece) {
      const int slot = lb <= piece * kLongRow ? 0 : 1;
      const vec_t t = *reinterpret_cast<const vec_t*>(ws + (piece * 2 + slot) * feat + col);
      float f[V];
      __builtin_memcpy(f, &t, sizeof(vec_t));
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] = reduce_op<RED>(acc[i], f[i]);
    }
  }
  if (RED == 3 && hb > lb)
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] /= (float)(hb - lb);
  if (col_ok && lane < L) {
    vec_t t;
    __builtin_memcpy(&t, acc, sizeof(vec_t));
    *reinterpret_cast<vec_t*>(out + r * feat + col) = t;
  }
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_gspmm_workspace_bytes(int64_t n_edges, int feat) {
  if (n_edges <= cxg::kLongRow || feat < 1) return 0;      // no row can be long
  return (size_t)cxg::ceil_div(n_edges, (int64_t)cxg::kLongRow) * 2 * (size_t)feat * sizeof(float);
}

int cxg_gspmm_i32_f32(const int32_t* rowptr, const int32_t* colind, const float* val, const float* b,
                      float* out, int64_t n_rows, int64_t n_edges, int feat, int reduce_op,
                      int compute_op, void* workspace, size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0 && feat >= 1, CXG_ERR_ARG, "bad n_rows/n_edges/feat");
  CXG_REQUIRE(n_edges < ((int64_t)1 << 31), CXG_ERR_ARG, "int32 CSR holds fewer than 2^31 edges");
  CXG_REQUIRE(reduce_op >= 0 && reduce_op <= 3, CXG_ERR_ARG, "reduce_op must be 0..3");
  CXG_REQUIRE(!val || (compute_op >= 0 && compute_op <= 3), CXG_ERR_ARG, "compute_op must be 0..3");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(rowptr && b && out, CXG_ERR_ARG, "null pointer");   // colind may be NULL for a graph without edges
  const size_t need = cxg_gspmm_workspace_bytes(n_edges, feat);
  CXG_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), CXG_ERR_ARG,
              "workspace smaller than cxg_gspmm_workspace_bytes");
  float* ws = reinterpret_cast<float*>(workspace);
  const float ini = reduce_op == 1 ? (float)INT_MIN : reduce_op == 2 ? (float)INT_MAX : 0.f;
  const bool wide = feat % 4 == 0 && (((uintptr_t)b | (uintptr_t)out | (uintptr_t)ws) & 15) == 0;
  const int slots = wide ? feat / 4 : feat;              // lanes a whole row would take
  int L = 1;
  while (L < slots && L < CXG_WAVE) L <<= 1;
  const int64_t n_pieces = need ? cxg::ceil_div(n_edges, (int64_t)cxg::kLongRow) : 0;
  const unsigned tiles = (unsigned)cxg::ceil_div(slots, L);
  const dim3 grid((unsigned)cxg::ceil_div(n_rows, cxg::kBlock / CXG_WAVE), tiles);
  const dim3 pgrid((unsigned)cxg::ceil_div(n_pieces, (int64_t)(cxg::kBlock / CXG_WAVE)), tiles);
  const dim3 block(cxg::kBlock);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define CXG_GSPMM_V(R, C, HV, V)                                                                     \
  do {                                                                                               \
    if (n_pieces)                                                                                    \
      hipLaunchKernelGGL((cxg::gspmm_long_rows_kernel<R, C, HV, V>), pgrid, block, 0, st, rowptr,   \
                         colind, val, b, ws, n_rows, n_pieces, feat, ini, L);                        \
    hipLaunchKernelGGL((cxg::gspmm_row_kernel<R, C, HV, V>), grid, block, 0, st, rowptr, colind,     \
                       val, b, out, ws, n_rows, feat, ini, L);                                       \
  } while (0)
#define CXG_GSPMM(R, C, HV)                                                                          \
  do {                                                                                               \
    if (wide) CXG_GSPMM_V(R, C, HV, 4);                                                              \
    else CXG_GSPMM_V(R, C, HV, 1);                                                                   \
  } while (0)
#define CXG_GSPMM_COMP(R)                                   \
  do {                                                      \
    if (!val) CXG_GSPMM(R, 0, false);                       \
    else if (compute_op == 0) CXG_GSPMM(R, 0, true);        \
    else if (compute_op == 1) CXG_GSPMM(R, 1, true);        \
    else if (compute_op == 2) CXG_GSPMM(R, 2, true);        \
    else CXG_GSPMM(R, 3, true);                             \
  } while (0)
  if (reduce_op == 0) CXG_GSPMM_COMP(0);
  else if (reduce_op == 1) CXG_GSPMM_COMP(1);
  else if (reduce_op == 2) CXG_GSPMM_COMP(2);
  else CXG_GSPMM_COMP(3);
#undef CXG_GSPMM_COMP
#undef CXG_GSPMM
#undef CXG_GSPMM_V
  CXG_LAUNCH_CHECK("gspmm_row_kernel");
  return CXG_OK;
}

}  // extern "C"
