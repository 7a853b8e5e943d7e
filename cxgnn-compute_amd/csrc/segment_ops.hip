// Edge-parallel row sums of narrow per-edge data (1..8 floats per edge):
//
//   out[r, 0..W) = sum over the edges k of row r of in[sel ? sel[k] : k, 0..W)
//
// This is the shape of the source-gradient of the edge softmax (a gather through
// the transposed graph's `perm`) and of spmv.  A wave-per-row or lane-per-row
// kernel leaves most lanes idle on power-law graphs; here every lane owns one
// edge, whatever its row's length:
//   * the edge array is cut into spans of T edges, one wave per span, 64 edges
//     per step; the row of every edge comes from a precomputed int32 row-id
//     array (4 bytes per edge, coalesced), so no per-row bookkeeping is needed;
//   * the 64 values of a step are summed per row by a segmented inclusive scan
//     across the lanes (six shuffle steps, segment starts from a ballot), and
//     the last lane of each row segment writes the row;
//   * a row that runs past a step is carried in registers, a row that runs past
//     a span leaves head / tail partials that a second small kernel adds in span
//     order -- no atomics, deterministic.
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;

constexpr int kRowSpan = 8 * CXG_WAVE;       // positions one wave expands

__global__ __launch_bounds__(256) void row_ids32_kernel(const int64_t* __restrict__ ptr, int64_t n_rows,
                                                        int64_t n_edges, int32_t* __restrict__ rows) {
  const int lane = lane_id();
  const int64_t w = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t k0 = uniform_i64(w * kRowSpan);
  if (k0 >= n_edges) return;
  RowWalker walk;
  walk.init(ptr, n_rows, ptr[0] + k0);
  for (int c = 0; c < kRowSpan; c += CXG_WAVE) {
    if (k0 + c >= n_edges) break;
    const int64_t k = k0 + c + lane;
    const int64_t row = walk.row_of(c + lane, k < n_edges);
    if (k < n_edges) rows[k] = (int32_t)row;
  }
}

__global__ void zero_f32_kernel(float* __restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

template <int W> __device__ __forceinline__ void load_w(const float* __restrict__ p, float (&v)[W]) {
  if constexpr (W == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else if constexpr (W == 2) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    v[0] = t.x; v[1] = t.y;
  } else if constexpr (W == 8) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    const float4 u = *reinterpret_cast<const float4*>(p + 4);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; v[4] = u.x; v[5] = u.y; v[6] = u.z; v[7] = u.w;
  } else {
#pragma unroll
    for (int i = 0; i < W; ++i) v[i] = p[i];
  }
}
template <int W> __device__ __forceinline__ void store_w(float* __restrict__ p, const float (&v)[W]) {
  if constexpr (W == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else if constexpr (W == 2) {
    *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
  } else if constexpr (W == 8) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int i = 0; i < W; ++i) p[i] = v[i];
  }
}

template <int W>
__global__ __launch_bounds__(kBlock) void segment_gather_sum_kernel(
    const int32_t* __restrict__ rows, const int64_t* __restrict__ ptr, const int64_t* __restrict__ sel,
    const float* __restrict__ in, float* __restrict__ out, int64_t n_edges, int T,
    float* __restrict__ carry, int64_t* __restrict__ tail_row) {
  const int lane = lane_id();
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + uniform_i32(threadIdx.x >> 6);
  const int64_t n_spans = (n_edges + T - 1) / T;
  if (s >= n_spans) return;
  const int64_t e0 = s * T;
  const int n = (int)((n_edges - e0) < (int64_t)T ? (n_edges - e0) : (int64_t)T);
  const int64_t e_begin = ptr[0];

  int prev_last = e0 > 0 ? rows[e0 - 1] : -1;      // row of the edge before lane 0 (wave-uniform)
  bool head_open = rows[e0] == prev_last;          // the span starts inside a row
  float carry_v[W];
#pragma unroll
  for (int w = 0; w < W; ++w) carry_v[w] = 0.f;
  bool open = head_open;                           // the last segment so far has not ended

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    const int64_t j = e0 + c0 + lane;
    const bool valid = lane < cn;
    const int rid = valid ? rows[j] : -1;
    int rid_next = __shfl_down(rid, 1);
    if (lane == cn - 1) rid_next = (j + 1 < n_edges) ? rows[j + 1] : -2;
    int rid_prev = __shfl_up(rid, 1);
    if (lane == 0) rid_prev = prev_last;
    const unsigned long long starts = __ballot(valid && rid != rid_prev) | 1ull;
    const bool cont0 = bcast_i32(rid, 0) == prev_last;   // lane 0 continues the previous segment

    float v[W];
#pragma unroll
    for (int w = 0; w < W; ++w) v[w] = 0.f;
    if (valid) {
      const int64_t pos = e_begin + j;
      load_w<W>(in + (sel ? sel[pos] : pos) * W, v);
    }
    // first lane of this lane's segment within the step
    const int seg0 = 63 - __clzll((long long)(starts & ((2ull << lane) - 1ull)));
#pragma unroll
    for (int off = 1; off < CXG_WAVE; off <<= 1) {
      const bool take = lane - off >= seg0;
#pragma unroll
      for (int w = 0; w < W; ++w) {
        const float u = __shfl_up(v[w], off);
        if (take) v[w] += u;
      }
    }
    const bool in_first = seg0 == 0;
    if (cont0 && in_first) {
#pragma unroll
      for (int w = 0; w < W; ++w) v[w] += carry_v[w];
    }
    const bool tail = valid && rid != rid_next;
    const bool head_seg = head_open && in_first;        // this segment is the row the span started in
    if (tail) {
      if (head_seg) store_w<W>(carry + (size_t)(2 * s) * W, v);
      else store_w<W>(out + (int64_t)rid * W, v);
    }
    if (__ballot(tail && head_seg)) head_open = false;
    const bool last_is_tail = (__ballot(tail) >> (cn - 1)) & 1ull;
    open = !last_is_tail;
#pragma unroll
    for (int w = 0; w < W; ++w) carry_v[w] = open ? bcast_f32(v[w], cn - 1) : 0.f;
    prev_last = bcast_i32(rid, cn - 1);
  }

  int64_t t = -1;
  if (open) {
    if (head_open) {
      if (lane == 0) store_w<W>(carry + (size_t)(2 * s) * W, carry_v);       // the row covers the whole span
    } else {
      if (lane == 0) store_w<W>(carry + (size_t)(2 * s + 1) * W, carry_v);
      t = prev_last;
    }
  }
  if (lane == 0) tail_row[s] = t;
}

// One thread per span that holds the tail partial of a row: add the head
// partials of the following spans the row runs through, in span order.
template <int W>
__global__ void segment_fixup_kernel(const int64_t* __restrict__ ptr, float* __restrict__ out,
                                     int64_t n_edges, int T, const float* __restrict__ carry,
                                     const int64_t* __restrict__ tail_row) {
  const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t n_spans = (n_edges + T - 1) / T;
  if (s >= n_spans) return;
  const int64_t t = tail_row[s];
  if (t < 0) return;
  const int64_t s_last = (ptr[t + 1] - 1 - ptr[0]) / T;
  float acc[W];
#pragma unroll
  for (int w = 0; w < W; ++w) acc[w] = carry[(size_t)(2 * s + 1) * W + w];
  for (int64_t q = s + 1; q <= s_last; ++q) {
#pragma unroll
    for (int w = 0; w < W; ++w) acc[w] += carry[(size_t)(2 * q) * W + w];
  }
#pragma unroll
  for (int w = 0; w < W; ++w) out[t * W + w] = acc[w];
}

int span_for(int64_t n_edges) {
  int64_t t = n_edges / 16384;
  t = (t + 63) / 64 * 64;
  if (t < 64) t = 64;
  if (t > 512) t = 512;
  return (int)t;
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_csr_row_ids_i32(const int64_t* ptr, int64_t n_rows, int64_t n_edges, int32_t* rows,
                        void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(n_rows < ((int64_t)1 << 31), CXG_ERR_UNSUPPORTED, "row ids do not fit int32");
  if (n_edges == 0) return CXG_OK;
  CXG_REQUIRE(ptr && rows, CXG_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(cxg::row_ids32_kernel,
                     dim3((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges, cxg::kRowSpan), 4)), dim3(256), 0,
                     reinterpret_cast<hipStream_t>(stream), ptr, n_rows, n_edges, rows);
  CXG_LAUNCH_CHECK("row_ids32_kernel");
  return CXG_OK;
}

size_t cxg_segment_gather_sum_workspace_bytes(int64_t n_edges, int width) {
  if (n_edges < 0 || width < 1) return 0;
  const int64_t n_spans = n_edges > 0 ? cxg::ceil_div(n_edges, cxg::span_for(n_edges)) : 1;
  return cxg::align256((size_t)n_spans * sizeof(int64_t)) +
         cxg::align256((size_t)n_spans * 2 * (size_t)width * sizeof(float)) + 256;
}

int cxg_segment_gather_sum_f32(const int32_t* rows, const int64_t* ptr, const int64_t* sel,
                               const float* in, float* out, int64_t n_rows, int64_t n_edges, int width,
                               void* workspace, size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(width == 1 || width == 2 || width == 4 || width == 8, CXG_ERR_UNSUPPORTED,
              "width must be 1, 2, 4 or 8");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(out && ptr, CXG_ERR_ARG, "null out/ptr");
  CXG_REQUIRE(n_edges == 0 || (rows && in), CXG_ERR_ARG, "null rows/in");
  CXG_REQUIRE(((uintptr_t)in & (4 * (size_t)width - 1)) == 0 && ((uintptr_t)out & (4 * (size_t)width - 1)) == 0,
              CXG_ERR_ARG, "in/out must be aligned to a whole item");
  const size_t need = cxg_segment_gather_sum_workspace_bytes(n_edges, width);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t total = n_rows * width;
  hipLaunchKernelGGL(cxg::zero_f32_kernel, dim3((unsigned)cxg::ceil_div(total, 256)), dim3(256), 0, st, out,
                     total);
  CXG_LAUNCH_CHECK("zero_f32_kernel");
  if (n_edges == 0) return CXG_OK;
  const int T = cxg::span_for(n_edges);
  const int64_t n_spans = cxg::ceil_div(n_edges, T);
  int64_t* tail_row = reinterpret_cast<int64_t*>(workspace);
  float* carry = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) +
                                          cxg::align256((size_t)n_spans * sizeof(int64_t)));
  const dim3 grid((unsigned)cxg::ceil_div(n_spans, cxg::kWavesPerBlock)), block(cxg::kBlock);
  const dim3 fgrid((unsigned)cxg::ceil_div(n_spans, 256)), fblock(256);
#define CXG_SEG(WW)                                                                                  \
  do {                                                                                               \
    hipLaunchKernelGGL(cxg::segment_gather_sum_kernel<WW>, grid, block, 0, st, rows, ptr, sel, in, out, \
                       n_edges, T, carry, tail_row);                                                 \
    hipLaunchKernelGGL(cxg::segment_fixup_kernel<WW>, fgrid, fblock, 0, st, ptr, out, n_edges, T, carry, \
                       tail_row);                                                                    \
  } while (0)
  if (width == 1) CXG_SEG(1);
  else if (width == 2) CXG_SEG(2);
  else if (width == 4) CXG_SEG(4);
  else CXG_SEG(8);
#undef CXG_SEG
  CXG_LAUNCH_CHECK("segment_gather_sum_kernel");
  return CXG_OK;
}

}  // extern "C"
