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
// at the end of the row.  Sum and mean without edge values are served by the edge-span
// SpMM kernel instead (the host wrapper routes them there); this kernel covers the
// combinations that kernel has no carry rule for.
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

template <int RED, int COMP, bool HASVAL, int V>
__global__ __launch_bounds__(kBlock) void gspmm_row_kernel(
    const int32_t* __restrict__ rowptr, const int32_t* __restrict__ colind,
    const float* __restrict__ val, const float* __restrict__ b, float* __restrict__ out,
    int64_t n_rows, int feat, float ini, int L) {
  using vec_t = typename GVec<V>::type;
  const int lane = lane_id();
  const int64_t r = (int64_t)blockIdx.x * (kBlock / CXG_WAVE) + uniform_i32(threadIdx.x >> 6);
  if (r >= n_rows) return;
  const int G = CXG_WAVE / L;              // edges per round
  const int es = lane / L, le = lane % L;
  const int col = (blockIdx.y * L + le) * V;
  const bool col_ok = col < feat;          // feat % V == 0: a lane's V columns exist together
  const int lb = rowptr[r], hb = rowptr[r + 1];
  float acc[V];
#pragma unroll
  for (int i = 0; i < V; ++i) acc[i] = hb > lb ? ini : 0.f;
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
  // combine the edge groups (every group started from the operator's identity)
  for (int m = L; m < CXG_WAVE; m <<= 1)
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = reduce_op<RED>(acc[i], __shfl_xor(acc[i], m, CXG_WAVE));
  if (RED == 3 && hb > lb)
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] /= (float)(hb - lb);
  if (col_ok && es == 0) {
    vec_t t;
    __builtin_memcpy(&t, acc, sizeof(vec_t));
    *reinterpret_cast<vec_t*>(out + r * feat + col) = t;
  }
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_gspmm_i32_f32(const int32_t* rowptr, const int32_t* colind, const float* val, const float* b,
                      float* out, int64_t n_rows, int feat, int reduce_op, int compute_op,
                      void* stream) {
  CXG_REQUIRE(n_rows >= 0 && feat >= 1, CXG_ERR_ARG, "bad n_rows/feat");
  CXG_REQUIRE(reduce_op >= 0 && reduce_op <= 3, CXG_ERR_ARG, "reduce_op must be 0..3");
  CXG_REQUIRE(!val || (compute_op >= 0 && compute_op <= 3), CXG_ERR_ARG, "compute_op must be 0..3");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(rowptr && b && out, CXG_ERR_ARG, "null pointer");   // colind may be NULL for a graph without edges
  const float ini = reduce_op == 1 ? (float)INT_MIN : reduce_op == 2 ? (float)INT_MAX : 0.f;
  const bool wide = feat % 4 == 0 && (((uintptr_t)b | (uintptr_t)out) & 15) == 0;
  const int slots = wide ? feat / 4 : feat;              // lanes a whole row would take
  int L = 1;
  while (L < slots && L < CXG_WAVE) L <<= 1;
  const dim3 grid((unsigned)cxg::ceil_div(n_rows, cxg::kBlock / CXG_WAVE),
                  (unsigned)cxg::ceil_div(slots, L));
  const dim3 block(cxg::kBlock);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define CXG_GSPMM(R, C, HV)                                                                          \
  do {                                                                                               \
    if (wide)                                                                                        \
      hipLaunchKernelGGL((cxg::gspmm_row_kernel<R, C, HV, 4>), grid, block, 0, st, rowptr, colind, val, b, \
                         out, n_rows, feat, ini, L);                                                 \
    else                                                                                             \
      hipLaunchKernelGGL((cxg::gspmm_row_kernel<R, C, HV, 1>), grid, block, 0, st, rowptr, colind, val, b, \
                         out, n_rows, feat, ini, L);                                                 \
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
  CXG_LAUNCH_CHECK("gspmm_row_kernel");
  return CXG_OK;
}

}  // extern "C"
