// Per-destination edge softmax (GAT attention) and other row reductions over
// narrow per-edge data (a few floats per edge) for gfx950.
//
// Work decomposition ("three-tier row blocks").  A block of 4 wavefronts owns 256
// consecutive rows, 64 per wave.
//   * rows of at most kShortDeg edges: one row per lane;
//   * rows of at most kWaveDeg edges: one row at a time by a whole wave, lanes
//     striding over the row's edges, wave reduction at the end;
//   * longer rows: one row at a time by the whole block (256 threads) with an LDS
//     reduction, so that a 17k-edge hub is a chain of ~70 steps instead of ~270.
// Power-law graphs have millions of degree-1..8 rows and a few hundred rows with
// more than 10k edges; each tier keeps its lanes busy on its share.
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
constexpr int kWaveDeg = 512;

__device__ __forceinline__ float wave_max(float v) {
  for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, CXG_WAVE));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  for (int m = 32; m > 0; m >>= 1) v += __shfl_xor(v, m, CXG_WAVE);
  return v;
}

// Cooperative scopes: the same row code runs with 64 lanes (one wave) or with the
// 256 threads of the block; `li`/`nl` enumerate the participants.
struct WaveScope {
  int li;
  static constexpr int nl = CXG_WAVE;
  __device__ __forceinline__ float max(float v) const { return wave_max(v); }
  __device__ __forceinline__ float sum(float v) const { return wave_sum(v); }
  __device__ __forceinline__ bool any(bool p) const { return __ballot(p) != 0; }
  __device__ __forceinline__ bool leader() const { return li == 0; }
};
struct BlockScope {
  int li;
  float* red;   // kWavesPerBlock floats of LDS
  static constexpr int nl = kBlock;
  template <bool MAX>
  __device__ __forceinline__ float reduce(float v) const {
    v = MAX ? wave_max(v) : wave_sum(v);
    __syncthreads();                      // previous use of `red` is over
    if ((li & 63) == 0) red[li >> 6] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < kWavesPerBlock; ++w) r = MAX ? fmaxf(r, red[w]) : r + red[w];
    return r;
  }
  __device__ __forceinline__ float max(float v) const { return reduce<true>(v); }
  __device__ __forceinline__ float sum(float v) const { return reduce<false>(v); }
  __device__ __forceinline__ bool any(bool p) const { return reduce<true>(p ? 1.f : 0.f) > 0.f; }
  __device__ __forceinline__ bool leader() const { return li == 0; }
};

// short_fn(r, begin, end): one lane per short row.  coop_fn(scope, r, begin, end):
// wave-uniform (WaveScope) or block-uniform (BlockScope) arguments.
template <class ShortFn, class CoopFn>
__device__ __forceinline__ void tiered_rows(const int64_t* __restrict__ ptr, int64_t n_rows,
                                            ShortFn short_fn, CoopFn coop_fn) {
  __shared__ unsigned long long s_very_long[kWavesPerBlock];
  __shared__ float s_red[kWavesPerBlock];
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const int64_t r = row0 + wave * CXG_WAVE + lane;
  const bool valid = r < n_rows;
  int64_t b = 0, e = 0;
  if (valid) { b = ptr[r]; e = ptr[r + 1]; }
  const int64_t deg = e - b;
  if (valid && deg <= kShortDeg) short_fn(r, b, e);
  uint64_t todo = __ballot(valid && deg > kShortDeg && deg <= kWaveDeg);
  const uint64_t very_long = __ballot(valid && deg > kWaveDeg);
  WaveScope ws{lane};
  while (todo) {
    const int l = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    coop_fn(ws, bcast_i64(r, l), bcast_i64(b, l), bcast_i64(e, l));
  }
  if (lane == 0) s_very_long[wave] = very_long;
  __syncthreads();
  BlockScope bs{(int)threadIdx.x, s_red};
  for (int w = 0; w < kWavesPerBlock; ++w) {
    unsigned long long m = s_very_long[w];
    while (m) {
      const int l = __ffsll(m) - 1;
      m &= m - 1;
      const int64_t rr = row0 + w * CXG_WAVE + l;
      coop_fn(bs, rr, (int64_t)ptr[rr], (int64_t)ptr[rr + 1]);
    }
  }
  __syncthreads();   // s_very_long / s_red are reused by the next call
}

__device__ __forceinline__ float leaky(float t, float slope) { return fmaxf(t, t * slope); }

// N consecutive floats / bytes starting at p, as one vector access where N allows
// (p is N*4-byte / N-byte aligned: the arrays are [*, N] with an aligned base).
template <int N> __device__ __forceinline__ void load_f(const float* __restrict__ p, float (&v)[N]) {
  if constexpr (N == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else if constexpr (N == 2) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    v[0] = t.x; v[1] = t.y;
  } else if constexpr (N == 8) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    const float4 u = *reinterpret_cast<const float4*>(p + 4);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; v[4] = u.x; v[5] = u.y; v[6] = u.z; v[7] = u.w;
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = p[i];
  }
}
template <int N> __device__ __forceinline__ void store_f(float* __restrict__ p, const float (&v)[N]) {
  if constexpr (N == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else if constexpr (N == 2) {
    *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
  } else if constexpr (N == 8) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = v[i];
  }
}
template <int N> __device__ __forceinline__ void load_b(const uint8_t* __restrict__ p, bool (&v)[N]) {
  if constexpr (N == 4 || N == 8) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      const uint32_t t = reinterpret_cast<const uint32_t*>(p)[w];
#pragma unroll
      for (int i = 0; i < 4; ++i) v[4 * w + i] = ((t >> (8 * i)) & 0xffu) != 0;
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = p[i] != 0;
  }
}
template <int N> __device__ __forceinline__ void store_b(uint8_t* __restrict__ p, const bool (&v)[N]) {
  if constexpr (N == 4 || N == 8) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      uint32_t t = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) t |= (v[4 * w + i] ? 1u : 0u) << (8 * i);
      reinterpret_cast<uint32_t*>(p)[w] = t;
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = v[i] ? 1 : 0;
  }
}

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
  // H > 0: compile-time head count; H == 0: runtime `heads`, one head at a time.
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;     // heads processed together
  for (int h0 = 0; h0 < nh; h0 += HB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float d[HB], m[HB], s[HB];
      load_f<HB>(att_dst + r * nh + h0, d);
#pragma unroll
      for (int h = 0; h < HB; ++h) { m[h] = kMaxInit; s[h] = 0.f; }
      for (int64_t k = b; k < e; ++k) {
        float as[HB];
        load_f<HB>(att_src + idx[k] * nh + h0, as);
#pragma unroll
        for (int h = 0; h < HB; ++h) online_add(m[h], s[h], leaky(d[h] + as[h], slope));
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = 1.0f / s[h];
      for (int64_t k = b; k < e; ++k) {
        float as[HB], o[HB];
        bool mk[HB];
        load_f<HB>(att_src + idx[k] * nh + h0, as);
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const float t = leaky(d[h] + as[h], slope);
          o[h] = __expf(t - m[h]) * s[h];
          mk[h] = t > 0.f;
        }
        store_f<HB>(out + k * nh + h0, o);
        store_b<HB>(mask + k * nh + h0, mk);
      }
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float d[HB], m[HB], s[HB];
      load_f<HB>(att_dst + r * nh + h0, d);
#pragma unroll
      for (int h = 0; h < HB; ++h) { m[h] = kMaxInit; s[h] = 0.f; }
      for (int64_t k = b + sc.li; k < e; k += sc.nl) {
        float as[HB];
        load_f<HB>(att_src + idx[k] * nh + h0, as);
#pragma unroll
        for (int h = 0; h < HB; ++h) online_add(m[h], s[h], leaky(d[h] + as[h], slope));
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) {
        const float mw = sc.max(m[h]);
        s[h] = 1.0f / sc.sum(s[h] * __expf(m[h] - mw));
        m[h] = mw;
      }
      for (int64_t k = b + sc.li; k < e; k += sc.nl) {
        float as[HB], o[HB];
        bool mk[HB];
        load_f<HB>(att_src + idx[k] * nh + h0, as);
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          const float t = leaky(d[h] + as[h], slope);
          o[h] = __expf(t - m[h]) * s[h];
          mk[h] = t > 0.f;
        }
        store_f<HB>(out + k * nh + h0, o);
        store_b<HB>(mask + k * nh + h0, mk);
      }
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

template <int H>
__global__ __launch_bounds__(kBlock) void edge_softmax_bwd_kernel(
    const int64_t* __restrict__ ptr, const float* __restrict__ out, const uint8_t* __restrict__ mask,
    const float* __restrict__ grad, float* __restrict__ g_dst, float* __restrict__ t_edge,
    int64_t n_rows, int heads, float slope) {
  const int nh = H > 0 ? H : heads;
  constexpr int HB = H > 0 ? H : 1;
  for (int h0 = 0; h0 < nh; h0 += HB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { s[h] = 0.f; dsum[h] = 0.f; pos[h] = 0; neg[h] = 0; }
      for (int64_t k = b; k < e; ++k)
      {
        float o[HB], g[HB];
        load_f<HB>(out + k * nh + h0, o);
        load_f<HB>(grad + k * nh + h0, g);
#pragma unroll
        for (int h = 0; h < HB; ++h) s[h] += o[h] * g[h];
      }
      for (int64_t k = b; k < e; ++k)
      {
        float o[HB], g[HB], tv[HB];
        bool mk[HB];
        load_f<HB>(out + k * nh + h0, o);
        load_f<HB>(grad + k * nh + h0, g);
        load_b<HB>(mask + k * nh + h0, mk);
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          float t = o[h] * (g[h] - s[h]);
          if (!mk[h]) { t *= slope; neg[h] = 1; } else { pos[h] = 1; }
          dsum[h] += t;
          tv[h] = t;
        }
        store_f<HB>(t_edge + k * nh + h0, tv);
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) g_dst[r * nh + h0 + h] = (pos[h] && neg[h]) ? dsum[h] : 0.f;
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float s[HB], dsum[HB];
      int pos[HB], neg[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) { s[h] = 0.f; dsum[h] = 0.f; pos[h] = 0; neg[h] = 0; }
      for (int64_t k = b + sc.li; k < e; k += sc.nl)
      {
        float o[HB], g[HB];
        load_f<HB>(out + k * nh + h0, o);
        load_f<HB>(grad + k * nh + h0, g);
#pragma unroll
        for (int h = 0; h < HB; ++h) s[h] += o[h] * g[h];
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) s[h] = sc.sum(s[h]);
      for (int64_t k = b + sc.li; k < e; k += sc.nl)
      {
        float o[HB], g[HB], tv[HB];
        bool mk[HB];
        load_f<HB>(out + k * nh + h0, o);
        load_f<HB>(grad + k * nh + h0, g);
        load_b<HB>(mask + k * nh + h0, mk);
#pragma unroll
        for (int h = 0; h < HB; ++h) {
          float t = o[h] * (g[h] - s[h]);
          if (!mk[h]) { t *= slope; neg[h] = 1; } else { pos[h] = 1; }
          dsum[h] += t;
          tv[h] = t;
        }
        store_f<HB>(t_edge + k * nh + h0, tv);
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) {
        const float total = sc.sum(dsum[h]);
        const bool both = sc.any(pos[h] != 0) && sc.any(neg[h] != 0);
        if (sc.leader()) g_dst[r * nh + h0 + h] = both ? total : 0.f;
      }
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

// out[r, 0..W) = sum_{k in row r} in[sel[k], 0..W)   (sel == nullptr: in[k]).
template <int W>
__global__ __launch_bounds__(kBlock) void narrow_gather_sum_kernel(
    const int64_t* __restrict__ ptr, const int64_t* __restrict__ sel, const float* __restrict__ in,
    float* __restrict__ out, int64_t n_rows, int width) {
  const int nw = W > 0 ? W : width;
  constexpr int WB = W > 0 ? W : 1;
  for (int w0 = 0; w0 < nw; w0 += WB) {
    auto short_fn = [&](int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b; k < e; ++k) {
        float p[WB];
        load_f<WB>(in + (sel ? sel[k] : k) * nw + w0, p);
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) out[r * nw + w0 + w] = acc[w];
    };
    auto coop_fn = [&](auto sc, int64_t r, int64_t b, int64_t e) {
      float acc[WB];
#pragma unroll
      for (int w = 0; w < WB; ++w) acc[w] = 0.f;
      for (int64_t k = b + sc.li; k < e; k += sc.nl) {
        float p[WB];
        load_f<WB>(in + (sel ? sel[k] : k) * nw + w0, p);
#pragma unroll
        for (int w = 0; w < WB; ++w) acc[w] += p[w];
      }
#pragma unroll
      for (int w = 0; w < WB; ++w) {
        const float total = sc.sum(acc[w]);
        if (sc.leader()) out[r * nw + w0 + w] = total;
      }
    };
    tiered_rows(ptr, n_rows, short_fn, coop_fn);
  }
}

dim3 row_grid(int64_t n_rows) { return dim3((unsigned)ceil_div(n_rows, kBlock)); }

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
