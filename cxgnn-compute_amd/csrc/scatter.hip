// Transposed aggregation by atomic scatter for gfx950:
//   gx[dstrow(e), :] += w(e) * g[row(e), :],   dstrow(e) = idx[e] (+ rel[e]*rel_stride)
// for every edge e of rows [0, n_rows).  This is what the reference's backward
// kernels do (gen_bwd_sum, src/cpp/src/aggr_kernel.cu:220-249; aggr_rel_bwd,
// src/cpp/src/rel_spmm.cu:72-104).  The library's main backward path gathers
// over a transposed CSR instead (deterministic, no atomics); this kernel serves
// callers that have no transposed graph -- the relational scatter of aggr_rel,
// whose destination row depends on the edge type -- and accumulates into the
// caller's buffer with hardware fp32 atomic adds.
//
// Edge spans as in the SpMM kernels: one wavefront per span of 256 consecutive
// edges; the gradient row of the current destination stays in registers while
// the wave walks that row's edges.
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;
constexpr int kSpan = 256;

struct ScatterArgs {
  const int64_t* ptr;
  const int64_t* idx;
  const int32_t* rel;
  int64_t rel_stride;
  const float* val;     // [E] or null
  const uint8_t* mask;  // [E] or null
  const float* g;       // [n_rows, feat]
  float* gx;            // [*, feat]
  int64_t n_rows;
  int feat;
};

__global__ __launch_bounds__(kBlock) void scatter_span_kernel(ScatterArgs a) {
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t e_begin = a.ptr[0];
  const int64_t e_end = a.ptr[a.n_rows];
  const int64_t e0 = e_begin + s * kSpan;
  if (e0 >= e_end) return;
  const int n = (int)((e_end - e0) < (int64_t)kSpan ? (e_end - e0) : (int64_t)kSpan);
  const int col = blockIdx.y * CXG_WAVE + lane;
  const bool col_ok = col < a.feat;
  int64_t r = wave_lower_bound(a.ptr, a.n_rows + 1, e0 + 1) - 1;   // row containing e0
  int64_t row_end = a.ptr[r + 1];
  float grow = col_ok ? a.g[r * a.feat + col] : 0.f;
  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_dst = -1;
    float my_w = 1.f;
    if (lane < cn) {
      const int64_t pos = e0 + c0 + lane;
      my_dst = a.idx[pos];
      if (a.rel) my_dst += (int64_t)a.rel[pos] * a.rel_stride;
      if (a.val) my_w = a.val[pos];
      if (a.mask && !a.mask[pos]) my_dst = -1;
    }
    for (int j = 0; j < cn; ++j) {
      const int64_t pos = e0 + c0 + j;
      while (pos >= row_end) {
        ++r;
        row_end = a.ptr[r + 1];
        if (pos < row_end) grow = col_ok ? a.g[r * a.feat + col] : 0.f;
      }
      const int64_t dst = bcast_i64(my_dst, j);
      const float w = bcast_f32(my_w, j);
      if (dst >= 0 && col_ok) unsafeAtomicAdd(a.gx + dst * a.feat + col, grow * w);
    }
  }
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_spmm_scatter_atomic_f32(const int64_t* ptr, const int64_t* idx, const int32_t* rel,
                                int64_t rel_stride, const float* val, const uint8_t* mask,
                                const float* g, float* gx, int64_t n_rows, int64_t n_edges_cap,
                                int feat, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges_cap >= 0 && feat >= 1, CXG_ERR_ARG, "bad sizes");
  if (n_rows == 0 || n_edges_cap == 0) return CXG_OK;
  CXG_REQUIRE(ptr && idx && g && gx, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(!rel || rel_stride > 0, CXG_ERR_ARG, "rel needs a positive rel_stride");
  cxg::ScatterArgs a;
  a.ptr = ptr; a.idx = idx; a.rel = rel; a.rel_stride = rel_stride; a.val = val; a.mask = mask;
  a.g = g; a.gx = gx; a.n_rows = n_rows; a.feat = feat;
  dim3 grid((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges_cap, cxg::kSpan), cxg::kWavesPerBlock),
            (unsigned)cxg::ceil_div(feat, CXG_WAVE));
  hipLaunchKernelGGL(cxg::scatter_span_kernel, grid, dim3(cxg::kBlock), 0,
                     reinterpret_cast<hipStream_t>(stream), a);
  CXG_LAUNCH_CHECK("scatter_span_kernel");
  return CXG_OK;
}

}  // extern "C"
