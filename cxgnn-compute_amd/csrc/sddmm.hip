// SDDMM for gfx950: per-edge dot products of a gathered source row with a
// destination row,   out[e,h] = sum_c a[src(e),h,c] * b[dst(e),(h,)c].
//
// Two entry points share the inner product code:
//   * CSR order (edges of a destination are consecutive): the destination row
//     is loaded once per row and kept in registers while the wave streams the
//     row's edges -- the reference's vertex-centric SDDMM
//     (src/cpp/src/sddmm_kernel.cu:27-278) and the edge-value gradient fused in
//     its weighted-SpMM backward (src/cpp/src/aggr_kernel.cu:321-361,443-491);
//   * COO order (explicit src/dst arrays): sddmm_multihead
//     (src/cpp/src/sddmm_kernel.cu:3-25).
// Work is cut into spans of consecutive edges, one wavefront per span, like the
// SpMM kernels; every output element is written exactly once (no atomics).
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * CXG_WAVE;
constexpr int kSpan = 256;

#ifndef CXG_SDDMM_U
#define CXG_SDDMM_U 16
#endif
#ifndef CXG_SDDMM_U_V4
#define CXG_SDDMM_U_V4 8
#endif
#ifndef CXG_SDDMM_COO_U
#define CXG_SDDMM_COO_U 8
#endif
#ifndef CXG_SDDMM_COO_U_V4
#define CXG_SDDMM_COO_U_V4 4
#endif

template <int V> struct Vec;
template <> struct Vec<1> { using type = float; };
template <> struct Vec<2> { using type = float2; };
template <> struct Vec<4> { using type = float4; };

__device__ __forceinline__ float vdot(float a, float b) { return a * b; }
__device__ __forceinline__ float vdot(float2 a, float2 b) { return a.x * b.x + a.y * b.y; }
__device__ __forceinline__ float vdot(float4 a, float4 b) {
  return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
template <int V> __device__ __forceinline__ typename Vec<V>::type vzero();
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }
template <> __device__ __forceinline__ float2 vzero<2>() { return make_float2(0.f, 0.f); }
template <> __device__ __forceinline__ float4 vzero<4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }

// Sum over aligned groups of `group` lanes (power of two <= 64); every lane of a
// group ends with the group's total.
// The first four butterfly steps stay inside a 16-lane DPP row and use data-parallel
// primitives (quad permutes and row mirrors, a few cycles each); only groups wider
// than a row need the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float group_sum(float v, int group) {
  if (group >= 2) v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]: lane ^ 1
  if (group >= 4) v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]: lane ^ 2
  if (group >= 8) v += dpp_f32<0x141>(v);   // row_half_mirror: the other quad of 8
  if (group >= 16) v += dpp_f32<0x140>(v);  // row_mirror: the other half of 16
  if (group >= 32) v += __shfl_xor(v, 16, CXG_WAVE);
  if (group >= 64) v += __shfl_xor(v, 32, CXG_WAVE);
  return v;
}

struct SddmmArgs {
  const int64_t* ptr;   // CSR form
  const int64_t* idx;
  const int64_t* src;   // COO form
  const int64_t* dst;
  const float* a;       // [n_src, heads, channels]
  const float* b;       // [n_dst, heads, channels] or [n_dst, channels]
  float* out;           // [n_edges, heads]
  int64_t n_rows, n_edges;
  int heads, channels;
  int b_heads;          // 1: b has a head dimension
  int group;            // lanes per head = channels / V   (packed kernels)
  // sddmm_multi_kernel only (a run of the heads of wider rows): floats between two rows
  // of a / b, floats between two rows of out
  int64_t lda, ldb;
  int ldo;
};

// Packed layout: the heads*channels floats of a row are spread over the 64 lanes,
// V consecutive floats per lane (heads*channels <= 64*V), `group` lanes per head.
template <int V>
__global__ __launch_bounds__(kBlock) void sddmm_csr_packed_kernel(SddmmArgs a) {
  using vec_t = typename Vec<V>::type;
  constexpr int U = (V == 4) ? CXG_SDDMM_U_V4 : CXG_SDDMM_U;
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t n_rows = a.n_rows;
  const int64_t e_begin = a.ptr[0];
  const int64_t e_end = a.ptr[n_rows];
  const int64_t e0 = e_begin + s * kSpan;
  if (e0 >= e_end) return;
  const int n = (int)((e_end - e0) < (int64_t)kSpan ? (e_end - e0) : (int64_t)kSpan);
  const int F = a.heads * a.channels;
  const int group = a.group;
  const bool active = lane * V < F;
  const int head = active ? (lane / group) : 0;
  const int bcol = a.b_heads ? lane * V : (lane % group) * V;
  const int64_t ldb = a.b_heads ? F : a.channels;
  const bool writer = active && (lane % group == 0);

  // row containing e0: last r with ptr[r] <= e0  (skip empty rows that start at e0)
  int64_t r = wave_lower_bound(a.ptr, n_rows + 1, e0 + 1) - 1;
  int64_t rbase = r;
  auto load_row_ends = [&](int64_t rb) -> int {
    int64_t q = rb + 1 + lane;
    if (q > n_rows) q = n_rows;
    const int64_t d = (int64_t)a.ptr[q] - e0;
    return (int)(d < (int64_t)n + 1 ? d : (int64_t)n + 1);
  };
  int row_ends = load_row_ends(rbase);
  int cur_end = bcast_i32(row_ends, 0);
  vec_t brow = active ? *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol) : vzero<V>();

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0;
    if (lane < cn) my_src = a.idx[e0 + c0 + lane];
    for (int b0 = 0; b0 < cn; b0 += U) {
      vec_t v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (b0 + u < cn) {
          const int64_t src = bcast_i64(my_src, b0 + u);
          v[u] = active ? *reinterpret_cast<const vec_t*>(a.a + src * F + lane * V) : vzero<V>();
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (b0 + u < cn) {
          const int j = c0 + b0 + u;
          while (j >= cur_end) {
            ++r;
            if (r - rbase == CXG_WAVE) { rbase = r; row_ends = load_row_ends(rbase); }
            cur_end = bcast_i32(row_ends, (int)(r - rbase));
            if (j < cur_end)
              brow = active ? *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol) : vzero<V>();
          }
          const float p = group_sum(vdot(v[u], brow), group);
          if (writer) a.out[(e0 + j) * a.heads + head] = p;
        }
      }
    }
  }
}

template <int V>
__global__ __launch_bounds__(kBlock) void sddmm_coo_packed_kernel(SddmmArgs a) {
  using vec_t = typename Vec<V>::type;
  constexpr int U = (V == 4) ? CXG_SDDMM_COO_U_V4 : CXG_SDDMM_COO_U;
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t e0 = s * kSpan;
  if (e0 >= a.n_edges) return;
  const int n = (int)((a.n_edges - e0) < (int64_t)kSpan ? (a.n_edges - e0) : (int64_t)kSpan);
  const int F = a.heads * a.channels;
  const int group = a.group;
  const bool active = lane * V < F;
  const int head = active ? (lane / group) : 0;
  const int bcol = a.b_heads ? lane * V : (lane % group) * V;
  const int64_t ldb = a.b_heads ? F : a.channels;
  const bool writer = active && (lane % group == 0);
  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0, my_dst = 0;
    if (lane < cn) { my_src = a.src[e0 + c0 + lane]; my_dst = a.dst[e0 + c0 + lane]; }
    for (int b0 = 0; b0 < cn; b0 += U) {
      vec_t va[U], vb[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (b0 + u < cn) {
          const int64_t src = bcast_i64(my_src, b0 + u);
          const int64_t dst = bcast_i64(my_dst, b0 + u);
          va[u] = active ? *reinterpret_cast<const vec_t*>(a.a + src * F + lane * V) : vzero<V>();
          vb[u] = active ? *reinterpret_cast<const vec_t*>(a.b + dst * ldb + bcol) : vzero<V>();
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (b0 + u < cn) {
          const float p = group_sum(vdot(va[u], vb[u]), group);
          if (writer) a.out[(e0 + c0 + b0 + u) * a.heads + head] = p;
        }
      }
    }
  }
}

// Tiled-output variants of the packed kernels for GROUP = channels / V in
// {8, 16, 32, 64} lanes per head.  After the lane-group reduction every lane of
// a group holds the (edge, head) product; instead of one 4-byte store per edge
// by the group leader (61.9M single-lane store instructions at the GAT shape),
// lane q of the group keeps the products of the edges q, GROUP + q, ... of the
// 64-edge step in registers, and the step ends with 64 / GROUP wave-wide stores
// that each cover 64 consecutive floats of `out`.
template <int V, int GROUP, bool COO>
__global__ __launch_bounds__(kBlock) void sddmm_tiled_kernel(SddmmArgs a) {
  using vec_t = typename Vec<V>::type;
  constexpr int S = CXG_WAVE / GROUP;                 // products kept per lane and step
  constexpr int U = COO ? 4 : (V == 4 ? 8 : 4);       // gathers in flight (measured optimum)
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t n_rows = a.n_rows;
  const int64_t e_begin = COO ? 0 : a.ptr[0];
  const int64_t e_end = COO ? a.n_edges : a.ptr[n_rows];
  const int64_t e0 = e_begin + s * kSpan;
  if (e0 >= e_end) return;
  const int n = (int)((e_end - e0) < (int64_t)kSpan ? (e_end - e0) : (int64_t)kSpan);
  const int F = a.heads * a.channels;
  const bool active = lane * V < F;
  const int head = lane / GROUP;
  const int q = lane % GROUP;
  const int bcol = a.b_heads ? lane * V : q * V;
  const int64_t ldb = a.b_heads ? F : a.channels;

  // CSR form: row containing e0 and the ends of the next 64 rows, relative to e0
  int64_t r = 0, rbase = 0;
  int row_ends = 0, cur_end = 0;
  vec_t brow = vzero<V>();
  auto load_row_ends = [&](int64_t rb) -> int {
    int64_t k = rb + 1 + lane;
    if (k > n_rows) k = n_rows;
    const int64_t d = (int64_t)a.ptr[k] - e0;
    return (int)(d < (int64_t)n + 1 ? d : (int64_t)n + 1);
  };
  if (!COO) {
    r = wave_lower_bound(a.ptr, n_rows + 1, e0 + 1) - 1;
    rbase = r;
    row_ends = load_row_ends(rbase);
    cur_end = bcast_i32(row_ends, 0);
    if (active) brow = *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol);
  }

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0, my_dst = 0;
    if (lane < cn) {
      my_src = COO ? a.src[e0 + c0 + lane] : a.idx[e0 + c0 + lane];
      if (COO) my_dst = a.dst[e0 + c0 + lane];
    }
    float res[S];
#pragma unroll
    for (int t = 0; t < S; ++t) res[t] = 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) {
      if (t * GROUP >= cn) break;
      for (int b0 = 0; b0 < GROUP; b0 += U) {
        vec_t va[U], vb[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int jj = t * GROUP + b0 + u;
          if (jj < cn) {
            const int64_t src = bcast_i64(my_src, jj);
            va[u] = active ? *reinterpret_cast<const vec_t*>(a.a + src * F + lane * V) : vzero<V>();
            if (COO) {
              const int64_t dst = bcast_i64(my_dst, jj);
              vb[u] = active ? *reinterpret_cast<const vec_t*>(a.b + dst * ldb + bcol) : vzero<V>();
            }
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int jj = t * GROUP + b0 + u;
          if (jj < cn) {
            if (!COO) {
              const int j = c0 + jj;
              while (j >= cur_end) {
                ++r;
                if (r - rbase == CXG_WAVE) { rbase = r; row_ends = load_row_ends(rbase); }
                cur_end = bcast_i32(row_ends, (int)(r - rbase));
                if (j < cur_end)
                  brow = active ? *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol) : vzero<V>();
              }
            }
            const float p = group_sum(vdot(va[u], COO ? vb[u] : brow), GROUP);
            if (q == b0 + u) res[t] = p;
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < S; ++t) {
      const int jj = t * GROUP + q;
      if (active && jj < cn) a.out[(e0 + c0 + jj) * a.heads + head] = res[t];
    }
  }
}

// Narrow rows (heads * channels <= 128 floats): several edges per gather
// instruction.  An edge occupies LE = heads * GROUP lanes (16 bytes each), the
// wave holds 64 / LE edge slots; one step gathers one source row per slot (CSR
// form: consecutive edges of the current destination row, whose row all slots
// share; COO form: every slot also fetches its own destination row).  The group
// leaders leave the products in a per-wave LDS tile of 64 x heads floats and each
// 64-edge step ends with coalesced stores from that tile.  One whole wave per edge
// left these shapes bound by one gather instruction per edge.
constexpr int kMultiMaxHeads = 8;

__device__ __forceinline__ int64_t sd_shfl_i64(int64_t v, int src_lane) {
  const int lo = __shfl((int)(v & 0xffffffffll), src_lane, CXG_WAVE);
  const int hi = __shfl((int)(v >> 32), src_lane, CXG_WAVE);
  return ((int64_t)hi << 32) | (uint32_t)lo;
}

template <int GROUP, bool COO>
__global__ __launch_bounds__(kBlock) void sddmm_multi_kernel(SddmmArgs a) {
  constexpr int V = 4;
  constexpr int UF = 4;                              // steps issued together
  using vec_t = typename Vec<V>::type;
  __shared__ float s_res[kWavesPerBlock][CXG_WAVE * kMultiMaxHeads];
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t n_rows = a.n_rows;
  const int64_t e_begin = COO ? 0 : a.ptr[0];
  const int64_t e_end = COO ? a.n_edges : a.ptr[n_rows];
  const int64_t e0 = e_begin + s * kSpan;
  if (e0 >= e_end) return;
  const int n = (int)((e_end - e0) < (int64_t)kSpan ? (e_end - e0) : (int64_t)kSpan);
  const int H = a.heads;
  const int F = H * a.channels;                      // = LE * V
  const int LE = H * GROUP;                          // lanes per edge (power of two <= 32)
  const int EPI = CXG_WAVE / LE;                     // edges per step
  const int es = lane / LE, le = lane % LE;
  const int head = le / GROUP, q = lane % GROUP;
  const int bcol = a.b_heads ? le * V : q * V;
  const int64_t lda = a.lda, ldb = a.ldb;
  const int ldo = a.ldo;
  float* const res = s_res[wave];

  int64_t r = 0, rbase = 0;
  int row_ends = 0, cur_end = 0;
  vec_t brow = vzero<V>();
  auto load_row_ends = [&](int64_t rb) -> int {
    int64_t k = rb + 1 + lane;
    if (k > n_rows) k = n_rows;
    const int64_t d = (int64_t)a.ptr[k] - e0;
    return (int)(d < (int64_t)n + 1 ? d : (int64_t)n + 1);
  };
  if (!COO) {
    r = wave_lower_bound(a.ptr, n_rows + 1, e0 + 1) - 1;
    rbase = r;
    row_ends = load_row_ends(rbase);
    cur_end = bcast_i32(row_ends, 0);
    brow = *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol);
  }

  for (int c0 = 0; c0 < n; c0 += CXG_WAVE) {
    const int cn = (n - c0) < CXG_WAVE ? (n - c0) : CXG_WAVE;
    int64_t my_src = 0, my_dst = 0;
    if (lane < cn) {
      // index streams and products are touched once: non-temporal, so that they do not push
      // gathered rows out of the L2
      my_src = stream_load((COO ? a.src : a.idx) + e0 + c0 + lane);
      if (COO) my_dst = stream_load(a.dst + e0 + c0 + lane);
    }
    auto fetch = [&](int jj, bool act, vec_t& va, vec_t& vb) {
      const int64_t src = sd_shfl_i64(my_src, jj & 63);
      va = act ? *reinterpret_cast<const vec_t*>(a.a + src * lda + le * V) : vzero<V>();
      if (COO) {
        const int64_t dst = sd_shfl_i64(my_dst, jj & 63);
        vb = act ? *reinterpret_cast<const vec_t*>(a.b + dst * ldb + bcol) : vzero<V>();
      }
    };
    int j = 0;
    while (j < cn) {
      if (!COO) {
        while (c0 + j >= cur_end) {
          ++r;
          if (r - rbase == CXG_WAVE) { rbase = r; row_ends = load_row_ends(rbase); }
          cur_end = bcast_i32(row_ends, (int)(r - rbase));
          if (c0 + j < cur_end) brow = *reinterpret_cast<const vec_t*>(a.b + r * ldb + bcol);
        }
      }
      int left = cn - j;
      if (!COO && cur_end - (c0 + j) < left) left = cur_end - (c0 + j);
      if (left >= UF * EPI) {
        vec_t va[UF], vb[UF];
#pragma unroll
        for (int u = 0; u < UF; ++u) fetch(j + u * EPI + es, true, va[u], vb[u]);
#pragma unroll
        for (int u = 0; u < UF; ++u) {
          const float p = group_sum(vdot(va[u], COO ? vb[u] : brow), GROUP);
          if (q == 0) res[(j + u * EPI + es) * H + head] = p;
        }
        j += UF * EPI;
      } else {
        const int take = left < EPI ? left : EPI;
        const bool act = es < take;
        vec_t va, vb;
        fetch(j + es, act, va, vb);
        const float p = group_sum(vdot(va, COO ? vb : brow), GROUP);
        if (q == 0 && act) res[(j + es) * H + head] = p;
        j += take;
      }
    }
    __builtin_amdgcn_wave_barrier();                 // the tile is complete (one wave, in-order LDS)
    if (ldo == H) {
      for (int i = lane; i < cn * H; i += CXG_WAVE) stream_store(a.out + (e0 + c0) * H + i, res[i]);
    } else {
      for (int i = lane; i < cn * H; i += CXG_WAVE) stream_store(a.out + (e0 + c0 + i / H) * ldo + i % H, res[i]);
    }
    __builtin_amdgcn_wave_barrier();                 // read before the next step overwrites it
  }
}

// General layout (any heads / channels): one wave-wide reduction per (edge, head).
// COO == false walks CSR rows (dst = row), COO == true reads src/dst arrays.
template <bool COO>
__global__ __launch_bounds__(kBlock) void sddmm_general_kernel(SddmmArgs a) {
  const int lane = lane_id();
  const int wave = uniform_i32(threadIdx.x >> 6);
  const int64_t s = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t e_begin = COO ? 0 : a.ptr[0];
  const int64_t e_end = COO ? a.n_edges : a.ptr[a.n_rows];
  const int64_t e0 = e_begin + s * kSpan;
  if (e0 >= e_end) return;
  const int n = (int)((e_end - e0) < (int64_t)kSpan ? (e_end - e0) : (int64_t)kSpan);
  const int C = a.channels, H = a.heads;
  int64_t r = 0;
  if (!COO) r = wave_lower_bound(a.ptr, a.n_rows + 1, e0 + 1) - 1;
  for (int j = 0; j < n; ++j) {
    const int64_t e = e0 + j;
    int64_t src, dst;
    if (COO) {
      src = a.src[e];
      dst = a.dst[e];
    } else {
      while (e >= a.ptr[r + 1]) ++r;
      src = a.idx[e];
      dst = r;
    }
    for (int h = 0; h < H; ++h) {
      const float* pa = a.a + (src * H + h) * C;
      const float* pb = a.b_heads ? a.b + (dst * H + h) * C : a.b + dst * C;
      float p = 0.f;
      for (int c = lane; c < C; c += CXG_WAVE) p += pa[c] * pb[c];
      p = group_sum(p, CXG_WAVE);
      if (lane == 0) a.out[e * H + h] = p;
    }
  }
}

bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

// Vector width for the packed kernels, or 0 if the shape needs the general one.
int packed_vec(const SddmmArgs& a) {
  const int F = a.heads * a.channels;
  const uintptr_t bits = (uintptr_t)a.a | (uintptr_t)a.b;
  for (int v = 1; v <= 4; v *= 2) {
    if (a.channels % v != 0) break;
    if ((bits & (uintptr_t)(4 * v - 1)) != 0) break;
    const int g = a.channels / v;
    if (F <= CXG_WAVE * v && is_pow2(g) && g <= CXG_WAVE) return v;
  }
  return 0;
}

// Launches the several-edges-per-step kernel when an edge fits 32 lanes of 16 bytes; wider
// rows whose heads can be cut into runs that fit go through it one run of heads at a
// time (a run reads its slice of every gathered row: two passes over the 512-byte halves
// of 1 KB rows take a little less time than one pass with a wave per edge, 7.7 against
// 8.0 ms on the GAT graph).
constexpr int kMultiMaxPasses = 8;

template <bool COO>
bool launch_multi(SddmmArgs a, dim3 grid, dim3 block, hipStream_t st) {
  const uintptr_t bits = (uintptr_t)a.a | (uintptr_t)a.b;
  if (a.channels % 4 != 0 || (bits & 15) != 0) return false;
  a.group = a.channels / 4;
  if (!is_pow2(a.group) || a.group > 32) return false;
  int run = 1;                                       // heads per pass
  while (run * 2 <= a.heads && a.heads % (run * 2) == 0 && run * 2 * a.group <= 32 && run * 2 <= kMultiMaxHeads)
    run *= 2;
  const int passes = a.heads / run;
  if (passes > kMultiMaxPasses) return false;
  const int heads = a.heads;
  a.lda = (int64_t)heads * a.channels;
  a.ldb = a.b_heads ? a.lda : a.channels;
  a.ldo = heads;
  a.heads = run;
  for (int p = 0; p < passes; ++p) {
#define CXG_MULTI(GG) \
  if (a.group == GG) hipLaunchKernelGGL((sddmm_multi_kernel<GG, COO>), grid, block, 0, st, a);
    CXG_MULTI(1) CXG_MULTI(2) CXG_MULTI(4) CXG_MULTI(8) CXG_MULTI(16) CXG_MULTI(32)
#undef CXG_MULTI
    a.a += (int64_t)run * a.channels;
    if (a.b_heads) a.b += (int64_t)run * a.channels;
    a.out += run;
  }
  return true;
}

// Launches the tiled-output kernel when the group width has an instantiation.
template <bool COO>
bool launch_tiled(const SddmmArgs& a, int v, dim3 grid, dim3 block, hipStream_t st) {
#define CXG_TILED(VV, GG)                                                                   \
  if (v == VV && a.group == GG) {                                                           \
    hipLaunchKernelGGL((sddmm_tiled_kernel<VV, GG, COO>), grid, block, 0, st, a);           \
    return true;                                                                            \
  }
  CXG_TILED(4, 8) CXG_TILED(4, 16) CXG_TILED(4, 32) CXG_TILED(4, 64)
  CXG_TILED(2, 8) CXG_TILED(2, 16) CXG_TILED(2, 32) CXG_TILED(2, 64)
  CXG_TILED(1, 8) CXG_TILED(1, 16) CXG_TILED(1, 32) CXG_TILED(1, 64)
#undef CXG_TILED
  return false;
}

int check_common(const float* a, const float* b, float* out, int heads, int channels) {
  CXG_REQUIRE(heads >= 1 && channels >= 1, CXG_ERR_ARG, "heads/channels must be >= 1");
  CXG_REQUIRE(a && b && out, CXG_ERR_ARG, "null feature/output pointer");
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_sddmm_csr_f32(const int64_t* ptr, const int64_t* idx, const float* src_feat,
                      const float* dst_feat, float* out, int64_t n_rows, int64_t n_edges_cap,
                      int heads, int channels, int dst_has_heads, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges_cap >= 0, CXG_ERR_ARG, "negative size");
  if (n_rows == 0 || n_edges_cap == 0) return CXG_OK;
  CXG_REQUIRE(ptr && idx, CXG_ERR_ARG, "null ptr/idx");
  int rc = cxg::check_common(src_feat, dst_feat, out, heads, channels);
  if (rc) return rc;
  cxg::SddmmArgs a{};
  a.ptr = ptr; a.idx = idx; a.a = src_feat; a.b = dst_feat; a.out = out;
  a.n_rows = n_rows; a.n_edges = n_edges_cap; a.heads = heads; a.channels = channels;
  a.b_heads = dst_has_heads ? 1 : 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges_cap, cxg::kSpan), cxg::kWavesPerBlock));
  dim3 block(cxg::kBlock);
  const int v = cxg::packed_vec(a);
  if (v) a.group = channels / v;
  if (cxg::launch_multi<false>(a, grid, block, st)) { /* several edges per step */ }
  else if (v && cxg::launch_tiled<false>(a, v, grid, block, st)) { /* coalesced-output form */ }
  else if (v == 4) hipLaunchKernelGGL(cxg::sddmm_csr_packed_kernel<4>, grid, block, 0, st, a);
  else if (v == 2) hipLaunchKernelGGL(cxg::sddmm_csr_packed_kernel<2>, grid, block, 0, st, a);
  else if (v == 1) hipLaunchKernelGGL(cxg::sddmm_csr_packed_kernel<1>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(cxg::sddmm_general_kernel<false>, grid, block, 0, st, a);
  CXG_LAUNCH_CHECK("sddmm_csr kernel");
  return CXG_OK;
}

int cxg_sddmm_coo_f32(const int64_t* src, const int64_t* dst, const float* src_feat,
                      const float* dst_feat, float* out, int64_t n_edges, int heads, int channels,
                      int dst_has_heads, void* stream) {
  CXG_REQUIRE(n_edges >= 0, CXG_ERR_ARG, "negative size");
  if (n_edges == 0) return CXG_OK;
  CXG_REQUIRE(src && dst, CXG_ERR_ARG, "null src/dst");
  int rc = cxg::check_common(src_feat, dst_feat, out, heads, channels);
  if (rc) return rc;
  cxg::SddmmArgs a{};
  a.src = src; a.dst = dst; a.a = src_feat; a.b = dst_feat; a.out = out;
  a.n_edges = n_edges; a.heads = heads; a.channels = channels;
  a.b_heads = dst_has_heads ? 1 : 0;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges, cxg::kSpan), cxg::kWavesPerBlock));
  dim3 block(cxg::kBlock);
  const int v = cxg::packed_vec(a);
  if (v) a.group = channels / v;
  if (cxg::launch_multi<true>(a, grid, block, st)) { /* several edges per step */ }
  else if (v && cxg::launch_tiled<true>(a, v, grid, block, st)) { /* coalesced-output form */ }
  else if (v == 4) hipLaunchKernelGGL(cxg::sddmm_coo_packed_kernel<4>, grid, block, 0, st, a);
  else if (v == 2) hipLaunchKernelGGL(cxg::sddmm_coo_packed_kernel<2>, grid, block, 0, st, a);
  else if (v == 1) hipLaunchKernelGGL(cxg::sddmm_coo_packed_kernel<1>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(cxg::sddmm_general_kernel<true>, grid, block, 0, st, a);
  CXG_LAUNCH_CHECK("sddmm_coo kernel");
  return CXG_OK;
}

}  // extern "C"
