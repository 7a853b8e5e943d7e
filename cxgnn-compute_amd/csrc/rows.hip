// Row-wise helpers for gfx950: copy rows by index, add rows into indexed
// destinations, and sum the head dimension of a [N, H, C] tensor.
//
//   scatter_add_rows : out[dest[e], :] += in[e, :]   gather_fwd, src/cpp/src/aggr.cu:42-51
//   gather_rows      : out[e, :] = in[sel[e], :]     gather_bwd, src/cpp/src/aggr.cu:53-62
//   head_sum         : out[n, c] = sum_h in[n, h, c] (the head reduction of
//                      spmm_multihead_pre_reduce, src/cpp/src/spmm_multihead_kernel.cu:3-36)
//
// Each wavefront moves whole rows with coalesced accesses; several rows are in
// flight per wave.  scatter_add_rows uses hardware fp32 atomic adds because
// several edges may target the same destination row (as the reference does).
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kBlock = 256;
constexpr int kRowsPerWave = 8;

template <bool SCATTER_ADD>
__global__ __launch_bounds__(kBlock) void rows_kernel(const float* __restrict__ in,
                                                      const int64_t* __restrict__ index,
                                                      float* __restrict__ out, int64_t n, int feat) {
  const int lane = lane_id();
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t e0 = wave * kRowsPerWave;
  for (int k = 0; k < kRowsPerWave; ++k) {
    const int64_t e = e0 + k;
    if (e >= n) return;
    const int64_t t = index[e];
    if (SCATTER_ADD) {
      const float* src = in + e * feat;
      float* dst = out + t * feat;
      for (int c = lane; c < feat; c += CXG_WAVE) unsafeAtomicAdd(dst + c, src[c]);
    } else {
      const float* src = in + t * feat;
      float* dst = out + e * feat;
      for (int c = lane; c < feat; c += CXG_WAVE) dst[c] = src[c];
    }
  }
}

// Rows of 1, 2, 4 or 8 floats: one row per thread as one (or two) vector accesses -- the
// stores of a wave are contiguous, the loads are the random part.  A wave per row would
// leave 60 of its 64 lanes idle on such rows.
template <int W>
__global__ __launch_bounds__(kBlock) void narrow_rows_gather_kernel(const float* __restrict__ in,
                                                                    const int64_t* __restrict__ sel,
                                                                    float* __restrict__ out, int64_t n) {
  const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (e >= n) return;
  const int64_t t = sel[e];
  if constexpr (W == 1) {
    out[e] = in[t];
  } else if constexpr (W == 2) {
    reinterpret_cast<float2*>(out)[e] = reinterpret_cast<const float2*>(in)[t];
  } else if constexpr (W == 4) {
    reinterpret_cast<float4*>(out)[e] = reinterpret_cast<const float4*>(in)[t];
  } else {
    const float4 a = reinterpret_cast<const float4*>(in)[2 * t], b = reinterpret_cast<const float4*>(in)[2 * t + 1];
    reinterpret_cast<float4*>(out)[2 * e] = a;
    reinterpret_cast<float4*>(out)[2 * e + 1] = b;
  }
}

__global__ __launch_bounds__(kBlock) void head_sum_kernel(const float* __restrict__ in,
                                                          float* __restrict__ out, int64_t n,
                                                          int heads, int channels) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * channels) return;
  const int64_t row = i / channels;
  const int c = (int)(i - row * channels);
  const float* p = in + row * heads * channels + c;
  float s = 0.f;
  for (int h = 0; h < heads; ++h) s += p[(int64_t)h * channels];
  out[i] = s;
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_scatter_add_rows_f32(const float* in, const int64_t* dest, float* out, int64_t n_edges,
                             int feat, void* stream) {
  CXG_REQUIRE(n_edges >= 0 && feat >= 1, CXG_ERR_ARG, "bad n_edges/feat");
  if (n_edges == 0) return CXG_OK;
  CXG_REQUIRE(in && dest && out, CXG_ERR_ARG, "null pointer");
  const int64_t waves = cxg::ceil_div(n_edges, cxg::kRowsPerWave);
  hipLaunchKernelGGL(cxg::rows_kernel<true>, dim3((unsigned)cxg::ceil_div(waves * CXG_WAVE, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), in, dest, out, n_edges,
                     feat);
  CXG_LAUNCH_CHECK("rows_kernel<scatter_add>");
  return CXG_OK;
}

int cxg_gather_rows_f32(const float* in, const int64_t* sel, float* out, int64_t n_rows_out, int feat,
                        void* stream) {
  CXG_REQUIRE(n_rows_out >= 0 && feat >= 1, CXG_ERR_ARG, "bad n_rows/feat");
  if (n_rows_out == 0) return CXG_OK;
  CXG_REQUIRE(in && sel && out, CXG_ERR_ARG, "null pointer");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool aligned = (((uintptr_t)in | (uintptr_t)out) & (uintptr_t)(feat >= 4 ? 15 : 4 * feat - 1)) == 0;
  if ((feat == 1 || feat == 2 || feat == 4 || feat == 8) && aligned) {
    const dim3 grid((unsigned)cxg::ceil_div(n_rows_out, cxg::kBlock)), block(cxg::kBlock);
    if (feat == 1) hipLaunchKernelGGL(cxg::narrow_rows_gather_kernel<1>, grid, block, 0, st, in, sel, out, n_rows_out);
    else if (feat == 2) hipLaunchKernelGGL(cxg::narrow_rows_gather_kernel<2>, grid, block, 0, st, in, sel, out, n_rows_out);
    else if (feat == 4) hipLaunchKernelGGL(cxg::narrow_rows_gather_kernel<4>, grid, block, 0, st, in, sel, out, n_rows_out);
    else hipLaunchKernelGGL(cxg::narrow_rows_gather_kernel<8>, grid, block, 0, st, in, sel, out, n_rows_out);
    CXG_LAUNCH_CHECK("narrow_rows_gather_kernel");
    return CXG_OK;
  }
  const int64_t waves = cxg::ceil_div(n_rows_out, cxg::kRowsPerWave);
  hipLaunchKernelGGL(cxg::rows_kernel<false>, dim3((unsigned)cxg::ceil_div(waves * CXG_WAVE, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), in, sel, out,
                     n_rows_out, feat);
  CXG_LAUNCH_CHECK("rows_kernel<gather>");
  return CXG_OK;
}

int cxg_head_sum_f32(const float* in, float* out, int64_t n_rows, int heads, int channels,
                     void* stream) {
  CXG_REQUIRE(n_rows >= 0 && heads >= 1 && channels >= 1, CXG_ERR_ARG, "bad shape");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(in && out, CXG_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(cxg::head_sum_kernel, dim3((unsigned)cxg::ceil_div(n_rows * channels, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), in, out, n_rows, heads,
                     channels);
  CXG_LAUNCH_CHECK("head_sum_kernel");
  return CXG_OK;
}

}  // extern "C"
