// Per-destination edge softmax (GAT attention) and other row reductions over
// narrow per-edge data (a few floats per edge) for gfx950.
//
// Work decomposition ("hybrid row blocks").  A wavefront owns 64 consecutive
// rows.  Rows of at most kShortDeg edges are handled one per lane; longer rows
// are then taken one at a time by the whole wave with lanes striding over the
// row's edges and a wave reduction at the end.  Power-law graphs have both
// millions of degree-1..8 rows and a few rows with >10k edges; this keeps the
// lanes busy on the former and bounds the serial chain on the latter.
//
//   forward  (edge_softmax_fwd, src/cpp/src/edge_softmax.cu:3-42):
//     t = leaky_relu(att_dst[r,h] + att_src[idx[e],h]);  out = softmax_row(t);
//     mask = t > 0.  Online max/sum in the first sweep, write in the second
//     (the reference makes three read-modify-write sweeps over out).
//   backward (edge_softmax_bwd, src/cpp/src/edge_softmax.cu:44-95):
//     s = sum_row out*g;  t = out*(g-s)*(mask ? 1 : slope);
//     g_dst[r,h] = sum_row t (left 0 unless the row has both signs, :91-93);
//     t is stored per edge and the source gradient is the row sum of t over the
//     transposed CSR (narrow_gather_sum below) instead of fp32 atomics.
//   spmv (spmv_csr, src/cpp/src/edge_softmax.cu:216-232) is narrow_gather_sum
//     with one float per edge.
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;
constexpr int kShortDeg = 16;

__device__ __forceinline__ float wave_max(float v) {
  for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, CXG_WAVE));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, CXG_WAVE);
  return v;
}

// Calls short_fn(r, begin, end) on one lane per short row, then long_fn(r, begin,
// end) with wave-uniform arguments for every long row of the wave's 64 rows.
template <class ShortFn, class LongFn>
__device__ __forceinline__ void hybrid_rows(const int64_t* __restrict__ ptr, int64_t n_rows,
                                            ShortFn short_fn, LongFn long_fn) {
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t r = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * CXG_WAVE + lane;
  const bool valid = r < n_rows;
  int64_t b = 0, e = 0;
  if (valid) { b = ptr[r]; e = ptr[r + 1]; }
  const bool is_long = valid && (e - b) > kShortDeg;
  if (valid && !is_long) short_fn(r, b, e);
  uint64_t todo = __ballot(is_long);
  while (todo) {
    const int l = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    long_fn(bcast_i64(r, l), bcast_i64(b, l), bcast_i64(e, l));
  }
}

__device__ __forceinline__ float leaky(float t, float slope) { return fmaxf(t, t * slope); }

// Online softmax state update: (m, s) <- combine with one value t.
__device__ __forceinline__ void online_add(float& m, float& s, float t) {
  const float mn = fmaxf(m, t);
  s = s * __expf(m - mn) + __expf(t - mn);
  m = mn;
}

constexpr float kMaxInit = -100000.f;  // running-max start of the reference kernel

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_fwd_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ idx,
    const float* __restrict__ att_dst, const float* __restrict__ att_src, float* __restrict__ out,
    uint8_t* __restrict__ mask, int64_t n_rows, int heads, float slope) {
  const int lane = lane_id();
  // H > 0: compile-time head count; H == 0: runtime `heads`, one head at a time.
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;     // heads processed together
  for (int h0 = 0; h0 < nh; h0 += HB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float d[HB], m[HB], s[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { d[h] = att_dst[r * nh + h0 + h]; m[h] = kMaxInit; s[h] = 0.f; }
      for (int64_t k = b; k < e; ++k) {
        const float* as = att_src + idx[k] * nh + h0;
#pragma unroll
        for (int h = 0; h < HB; ++h) online_add(m[h], s[h], leaky(d[h] + as[h], slope));
      }
      for (int64_t k = b; k < e; ++k) {
        const float* as = att_src + idx[k] * nh + h0;
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const float t = leaky(d[h] + as[h], slope);
          out[k * nh + h0 + h] = __expf(t - m[h]) / s[h];
          mask[k * nh + h0 + h] = t > 0.f;
        }
      }
    };
    auto long_fn = [&](int64_t r, int64_t b, int64_t e) {
      float d[HB], m[HB], s[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { d[h] = att_dst[r * nh + h0 + h]; m[h] = kMaxInit; s[h] = 0.f; }
      for (int64_t k = b + lane; k < e; k += CXG_WAVE) {
        const float* as = att_src + idx[k] * nh + h0;
#pragma unroll
        for (int h = 0; h < HB; ++h) online_add(m[h], s[h], leaky(d[h] + as[h], slope));
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) {
        const float mw = wave_max(m[h]);
        s[h] = wave_sum(s[h] * __expf(m[h] - mw));
        m[h] = mw;
      }
      for (int64_t k = b + lane; k < e; k += CXG_WAVE) {
        const float* as = att_src + idx[k] * nh + h0;
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const float t = leaky(d[h] + as[h], slope);
          out[k * nh + h0 + h] = __expf(t - m[h]) / s[h];
          mask[k * nh + h0 + h] = t > 0.f;
        }
      }
    };
    hybrid_rows(ptr, n_rows, short_fn, long_fn);
  }
}

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_bwd_kernel(
    const int64_t* __restrict__ ptr, const float* __restrict__ out, const uint8_t* __restrict__ mask,
    const float* __restrict__ grad, float* __restrict__ g_dst, float* __restrict__ t_edge,
    int64_t n_rows, int heads, float slope) {
  const int lane = lane_id();
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;
  for (int h0 = 0; h0 < nh; h0 += HB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { s[h] = 0.f; dsum[h] = 0.f; pos[h] = 0; neg[h] = 0; }
      for (int64_t k = b; k < e; ++k)
#pragma unroll
        for (int h = 0; h < HB; ++h) s[h] += out[k * nh + h0 + h] * grad[k * nh + h0 + h];
      for (int64_t k = b; k < e; ++k)
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const int64_t q = k * nh + h0 + h;
          float t = out[q] * (grad[q] - s[h]);
          if (!mask[q]) { t *= slope; neg[h] = 1; } else { pos[h] = 1; }
          dsum[h] += t;
          t_edge[q] = t;
        }
#pragma unroll
      for (int h = 0; h < HB; ++h) g_dst[r * nh + h0 + h] = (pos[h] && neg[h]) ? dsum[h] : 0.f;
    };
    auto long_fn = [&](int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { s[h] = 0.f; dsum[h] = 0.f; pos[h] = 0; neg[h] = 0; }
      for (int64_t k = b + lane; k < e; k += CXG_WAVE)
#pragma unroll
        for (int h = 0; h < HB; ++h) s[h] += out[k * nh + h0 + h] * grad[k * nh + h0 + h];
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = wave_sum(s[h]);
      for (int64_t k = b + lane; k < e; k += CXG_WAVE)
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const int64_t q = k * nh + h0 + h;
          float t = out[q] * (grad[q] - s[h]);
          if (!mask[q]) { t *= slope; neg[h] = 1; } else { pos[h] = 1; }
          dsum[h] += t;
          t_edge[q] = t;
        }
#pragma unroll
      for (int h = 0; h < HB; ++h) {
        const float total = wave_sum(dsum[h]);
        const bool both = (__ballot(pos[h] != 0) != 0) && (__ballot(neg[h] != 0) != 0);
        if (lane == 0) g_dst[r * nh + h0 + h] = both ? total : 0.f;
      }
    };
    hybrid_rows(ptr, n_rows, short_fn, long_fn);
  }
}

// out[r, 0..W) = sum_{k in row r} in[sel[k], 0..W)   (sel == nullptr: in[k]).
template <int W>
__global__ __launch_bounds__(kBlock) void narrow_gather_sum_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ sel, const float* __restrict__ in,
    float* __restrict__ out, int64_t n_rows, int width) {
  const int lane = lane_id();
  const int nw = W > 0 ? W : width;
  constexpr int WB = W > 0 ? W : 1;
  for (int w0 = 0; w0 < nw; w0 += WB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b; k < e; ++k) {
        const float* p = in + (sel ? sel[k] : k) * nw + w0;
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) out[r * nw + w0 + w] = acc[w];
    };
    auto long_fn = [&](int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b + lane; k < e; k += CXG_WAVE) {
        const float* p = in + (sel ? sel[k] : k) * nw + w0;
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) {
        const float total = wave_sum(acc[w]);
        if (lane == 0) out[r * nw + w0 + w] = total;
      }
    };
    hybrid_rows(ptr, n_rows, short_fn, long_fn);
  }
}

dim3 row_grid(int64_t n_rows) {
  return dim3((unsigned)ceil_div(ceil_div(n_rows, CXG_WAVE), kWavesPerBlock));
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_edge_softmax_fwd_f32(const int64_t* ptr, const int64_t* idx, const float* att_dst,
                             const float* att_src, float* out, uint8_t* mask, int64_t n_dst,
                             int heads, float slope, void* stream) {
  CXG_REQUIRE(n_dst >= 0 && heads >= 1, CXG_ERR_ARG, "bad n_dst/heads");
  if (n_dst == 0) return CXG_OK;
  CXG_REQUIRE(ptr && att_dst, CXG_ERR_ARG, "null ptr/att_dst");
  CXG_REQUIRE(idx && att_src && out && mask, CXG_ERR_ARG, "null idx/att_src/out/mask");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_dst), block(cxg::kBlock);
#define CXG_FWD(HH)                                                                         \
  hipLaunchKernelGGL(cxg::edge_softmax_fwd_kernel<HH>, grid, block, 0, st, ptr, idx, att_dst, \
                     att_src, out, mask, n_dst, heads, slope)
  if (heads == 1) CXG_FWD(1);
  else if (heads == 2) CXG_FWD(2);
  else if (heads == 4) CXG_FWD(4);
  else if (heads == 8) CXG_FWD(8);
  else CXG_FWD(0);
#undef CXG_FWD
  CXG_LAUNCH_CHECK("edge_softmax_fwd_kernel");
  return CXG_OK;
}

int cxg_edge_softmax_bwd_f32(const int64_t* ptr, const float* out, const uint8_t* mask,
                             const float* grad, float* g_dst, float* t_edge, int64_t n_dst, int heads,
                             float slope, void* stream) {
  CXG_REQUIRE(n_dst >= 0 && heads >= 1, CXG_ERR_ARG, "bad n_dst/heads");
  if (n_dst == 0) return CXG_OK;
  CXG_REQUIRE(ptr && g_dst, CXG_ERR_ARG, "null ptr/g_dst");
  CXG_REQUIRE(out && mask && grad && t_edge, CXG_ERR_ARG, "null out/mask/grad/t_edge");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_dst), block(cxg::kBlock);
#define CXG_BWD(HH)                                                                          \
  hipLaunchKernelGGL(cxg::edge_softmax_bwd_kernel<HH>, grid, block, 0, st, ptr, out, mask, grad, \
                     g_dst, t_edge, n_dst, heads, slope)
  if (heads == 1) CXG_BWD(1);
  else if (heads == 2) CXG_BWD(2);
  else if (heads == 4) CXG_BWD(4);
  else if (heads == 8) CXG_BWD(8);
  else CXG_BWD(0);
#undef CXG_BWD
  CXG_LAUNCH_CHECK("edge_softmax_bwd_kernel");
  return CXG_OK;
}

int cxg_narrow_gather_sum_f32(const int64_t* ptr, const int64_t* sel, const float* in, float* out,
                              int64_t n_rows, int width, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && width >= 1, CXG_ERR_ARG, "bad n_rows/width");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out, CXG_ERR_ARG, "null ptr/out");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid = cxg::row_grid(n_rows), block(cxg::kBlock);
#define CXG_NGS(WW)                                                                          \
  hipLaunchKernelGGL(cxg::narrow_gather_sum_kernel<WW>, grid, block, 0, st, ptr, sel, in, out, \
                     n_rows, width)
  if (width == 1) CXG_NGS(1);
  else if (width == 2) CXG_NGS(2);
  else if (width == 4) CXG_NGS(4);
  else if (width == 8) CXG_NGS(8);
  else CXG_NGS(0);
#undef CXG_NGS
  CXG_LAUNCH_CHECK("narrow_gather_sum_kernel");
  return CXG_OK;
}

}  // extern "C"
