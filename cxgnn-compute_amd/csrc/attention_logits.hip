// Per-node attention logits of a multi-head GAT layer and their gradients:
//   out_src[n,h] = sum_c x[n,h,c] * att_src[h,c]      (every source node)
//   out_dst[n,h] = sum_c x[n,h,c] * att_dst[h,c]      (the first n_dst nodes)
// (upstream computes both with broadcast multiplies and sums over the last axis,
// cxgnncomp/graph_conv.py:466-467).  Both logits come from one pass over x; the
// backward pass reads x once more and produces grad_x and both parameter gradients.
//
// Layout: a row of x is F = heads*channels floats, cut into S = F/V slots of V floats.
// A block holds S * rpb threads; thread t owns slot t % S for rows
// t/S, t/S + rpb, ... of the block's contiguous run of rows.  Consecutive threads read consecutive
// 16-byte pieces of consecutive rows, and a thread's (head, channel) never changes, so
// the parameter gradients accumulate in registers.  They leave the block through LDS
// (summed over the rpb row offsets in a fixed order) as one partial row per block; a
// second kernel sums the partial rows in block order.  The grid size depends on the
// shape only, hence results are reproducible bit for bit.
#include "cxg_common.hpp"

namespace cxg {
namespace {

#ifndef CXG_ATT_BLOCKS
#define CXG_ATT_BLOCKS 2048
#endif
#ifndef CXG_ATT_ROWS
#define CXG_ATT_ROWS 4
#endif
#ifndef CXG_ATT_THREADS
#define CXG_ATT_THREADS 256
#endif
constexpr int kMaxBlocks = CXG_ATT_BLOCKS;
constexpr int kMaxThreads = 1024;
constexpr int kTargetThreads = CXG_ATT_THREADS;
constexpr int kRowsInFlight = CXG_ATT_ROWS;          // rows a thread loads before it uses the first

template <int V> struct Vec;
template <> struct Vec<1> { using type = float; };
template <> struct Vec<2> { using type = float2; };
template <> struct Vec<4> { using type = float4; };

__device__ __forceinline__ float vdot(float a, float b) { return a * b; }
__device__ __forceinline__ float vdot(float2 a, float2 b) { return a.x * b.x + a.y * b.y; }
__device__ __forceinline__ float vdot(float4 a, float4 b) {
  return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
__device__ __forceinline__ float axpby(float s, float a, float t, float b) { return s * a + t * b; }
__device__ __forceinline__ float4 axpby(float s, float4 a, float t, float4 b) {
  return make_float4(s * a.x + t * b.x, s * a.y + t * b.y, s * a.z + t * b.z, s * a.w + t * b.w);
}
__device__ __forceinline__ void fma_into(float& acc, float s, float v) { acc += s * v; }
__device__ __forceinline__ void fma_into(float4& acc, float s, float4 v) {
  acc.x += s * v.x; acc.y += s * v.y; acc.z += s * v.z; acc.w += s * v.w;
}
template <int V> __device__ __forceinline__ typename Vec<V>::type vzero();
template <> __device__ __forceinline__ float vzero<1>() { return 0.f; }
template <> __device__ __forceinline__ float2 vzero<2>() { return make_float2(0.f, 0.f); }
template <> __device__ __forceinline__ float4 vzero<4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }

// Sum over `group` consecutive lanes (power of two <= 64, aligned); every lane of the
// group gets the total.
__device__ __forceinline__ float group_sum(float v, int group) {
  for (int m = 1; m < group; m <<= 1) v += __shfl_xor(v, m, CXG_WAVE);
  return v;
}

struct AttArgs {
  const float* x;          // [n_src, heads, channels]
  const float* att_src;    // [heads, channels]
  const float* att_dst;
  const float* g_src;      // [n_src, heads]   (backward)
  const float* g_dst;      // [n_dst, heads]
  float* out_src;          // [n_src, heads]   (forward)
  float* out_dst;          // [n_dst, heads]
  float* grad_x;           // [n_src, heads, channels]
  float* partial;          // [blocks, 2, F]
  int64_t n_src, n_dst;
  int heads, channels;
  int slots, rpb;          // F / V, rows per block step
  int64_t rows_per_block;  // contiguous rows one block walks
};

template <int V>
__global__ void att_logits_fwd_kernel(AttArgs a) {
  using vec_t = typename Vec<V>::type;
  const int j = threadIdx.x % a.slots, ro = threadIdx.x / a.slots;
  const int group = a.channels / V;
  const int h = j / group, q = j % group;
  const int64_t F = (int64_t)a.heads * a.channels;
  const vec_t as = *reinterpret_cast<const vec_t*>(a.att_src + j * V);
  const vec_t ad = *reinterpret_cast<const vec_t*>(a.att_dst + j * V);
  const int64_t stride = a.rpb;
  const int64_t begin = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t end = (begin + a.rows_per_block) < a.n_src ? (begin + a.rows_per_block) : a.n_src;
  for (int64_t n0 = begin + ro; n0 < end; n0 += kRowsInFlight * stride) {
    vec_t xv[kRowsInFlight];
#pragma unroll
    for (int u = 0; u < kRowsInFlight; ++u) {
      const int64_t n = n0 + u * stride;
      xv[u] = n < end ? *reinterpret_cast<const vec_t*>(a.x + n * F + j * V) : vzero<V>();
    }
#pragma unroll
    for (int u = 0; u < kRowsInFlight; ++u) {
      const int64_t n = n0 + u * stride;
      const float ps = group_sum(vdot(xv[u], as), group);
      const float pd = group_sum(vdot(xv[u], ad), group);
      if (q == 0 && n < end) {
        a.out_src[n * a.heads + h] = ps;
        if (n < a.n_dst) a.out_dst[n * a.heads + h] = pd;
      }
    }
  }
}

// Any shape: one thread per (node, head).
__global__ void att_logits_fwd_generic_kernel(AttArgs a) {
  const int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (u >= a.n_src * a.heads) return;
  const int h = (int)(u % a.heads);
  const int64_t n = u / a.heads;
  const float* xr = a.x + u * a.channels;
  const float* as = a.att_src + (int64_t)h * a.channels;
  const float* ad = a.att_dst + (int64_t)h * a.channels;
  float ps = 0.f, pd = 0.f;
  for (int c = 0; c < a.channels; ++c) {
    ps += xr[c] * as[c];
    pd += xr[c] * ad[c];
  }
  a.out_src[u] = ps;
  if (n < a.n_dst) a.out_dst[u] = pd;
}

template <int V, bool ACC>
__global__ void att_logits_bwd_kernel(AttArgs a) {
  using vec_t = typename Vec<V>::type;
  extern __shared__ float s_part[];            // [2][blockDim][V]
  const int j = threadIdx.x % a.slots, ro = threadIdx.x / a.slots;
  const int h = (j * V) / a.channels;
  const int64_t F = (int64_t)a.heads * a.channels;
  const vec_t as = *reinterpret_cast<const vec_t*>(a.att_src + j * V);
  const vec_t ad = *reinterpret_cast<const vec_t*>(a.att_dst + j * V);
  vec_t acc_s = vzero<V>(), acc_d = vzero<V>();
  const int64_t stride = a.rpb;
  const int64_t begin = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t end = (begin + a.rows_per_block) < a.n_src ? (begin + a.rows_per_block) : a.n_src;
  for (int64_t n0 = begin + ro; n0 < end; n0 += kRowsInFlight * stride) {
    vec_t xv[kRowsInFlight], old[kRowsInFlight];
    float gs[kRowsInFlight], gd[kRowsInFlight];
#pragma unroll
    for (int u = 0; u < kRowsInFlight; ++u) {
      const int64_t n = n0 + u * stride;
      const bool in = n < end;
      xv[u] = in ? *reinterpret_cast<const vec_t*>(a.x + n * F + j * V) : vzero<V>();
      if (ACC) old[u] = in ? *reinterpret_cast<const vec_t*>(a.grad_x + n * F + j * V) : vzero<V>();
      gs[u] = in ? a.g_src[n * a.heads + h] : 0.f;
      gd[u] = (in && n < a.n_dst) ? a.g_dst[n * a.heads + h] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kRowsInFlight; ++u) {
      const int64_t n = n0 + u * stride;
      if (n < end) {
        vec_t gx = axpby(gs[u], as, gd[u], ad);
        if (ACC) fma_into(gx, 1.f, old[u]);
        *reinterpret_cast<vec_t*>(a.grad_x + n * F + j * V) = gx;
      }
      fma_into(acc_s, gs[u], xv[u]);
      fma_into(acc_d, gd[u], xv[u]);
    }
  }
  vec_t* part = reinterpret_cast<vec_t*>(s_part);
  part[threadIdx.x] = acc_s;
  part[blockDim.x + threadIdx.x] = acc_d;
  __syncthreads();
  if (ro == 0) {
    vec_t ts = part[j], td = part[blockDim.x + j];
    for (int r = 1; r < a.rpb; ++r) {
      fma_into(ts, 1.f, part[r * a.slots + j]);
      fma_into(td, 1.f, part[blockDim.x + r * a.slots + j]);
    }
    float* row = a.partial + (int64_t)blockIdx.x * 2 * F;
    *reinterpret_cast<vec_t*>(row + j * V) = ts;
    *reinterpret_cast<vec_t*>(row + F + j * V) = td;
  }
}

// ---- Logits from the layer's input ---------------------------------------------------
// The transformed features are xs = x_in W^T, so both logits are linear in x_in:
//   out_src[n, h] = x_in[n, :] . m[h, :],      m[h, :]     = sum_c att_src[h, c] W[h*C + c, :]
//   out_dst[n, h] = x_in[n, :] . m[H + h, :],  m[H + h, :] = sum_c att_dst[h, c] W[h*C + c, :]
// (the contraction order of upstream's single-head einsum "mn,nho,ho->mh",
// cxgnncomp/graph_conv.py:500-511).  Where x_in is narrower than xs these kernels read
// fewer bytes per node, and in the backward pass the gradient of xs needs no second
// read-add-store pass: the logits' share goes to grad_x_in (rank 2H) and to grad_m.
//
// A row of x_in is `in` floats = S slots of 4; a group of G lanes (power of two >= S and
// >= J = 2H) walks one row, lanes at or past S hold zeros.  A lane keeps its 4 columns of
// all J rows of m in registers.  The J partial dot products of a row are folded over the
// group by halving: at lane distance G/2 a lane keeps one half of its values and sends
// the other, and so on, so that after log2 J steps a lane holds one value, which plain
// butterfly steps finish; lane q ends with value q / (G/J).
struct ProjArgs {
  const float* x;          // [n_src, in], row stride ldx
  const float* m;          // [J, in]
  const float* g_src;      // [n_src, H]   (backward)
  const float* g_dst;      // [n_dst, H]
  float* out_src;          // [n_src, H]   (forward)
  float* out_dst;          // [n_dst, H]
  float* grad_x;           // [n_src, in], row stride ldg
  float* partial;          // [blocks, J, in]
  int64_t ldx, ldg;
  int64_t n_src, n_dst;
  int in, slots, group, rpb;
  int64_t rows_per_block;
};

constexpr int kProjThreads = 256;

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }

// The partner lane's value at level M of the fold.  Levels below 16 stay inside a row of 16
// lanes and use data-parallel moves: rotate by 8, mirror the half row, reverse the quad,
// swap neighbours.  These pair lane l with l^8, l^7, l^3, l^1: each flips bit log2 M of
// the lane number and none of the higher bits, and together they reach every lane of the
// row, which is all the fold needs.
template <int M> __device__ __forceinline__ float lane_partner(float v) {
  static_assert(M == 8 || M == 4 || M == 2 || M == 1, "level inside a row of 16 lanes");
  constexpr int ctrl = M == 8 ? 0x128 : M == 4 ? 0x141 : M == 2 ? 0x1B : 0xB1;
  return __uint_as_float((unsigned)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), ctrl, 0xf, 0xf, true));
}

// lo + hi across the two rows (M = 16) or wave halves (M = 32) of a pair: the half-swap
// instructions exchange the odd rows (upper half) of their first operand with the even
// rows (lower half) of their second, after which the lower lane of a pair holds both
// `lo` values and the upper lane both `hi` values.
template <int M> __device__ __forceinline__ float swap_sum(float lo, float hi) {
  typedef unsigned v2u __attribute__((ext_vector_type(2)));
  static_assert(M == 16 || M == 32, "level across rows");
  const v2u r = M == 32 ? __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false)
                        : __builtin_amdgcn_permlane16_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
  return __uint_as_float(r.x) + __uint_as_float(r.y);
}

// Sums p[0..CNT) over a group of 2M lanes: while more than one value is left, a lane whose
// bit M is clear keeps the lower half of its values and its partner the upper half; lane q
// of a group of G lanes ends with the total of value q / (G / J) in p[0].
template <int CNT, int M> __device__ __forceinline__ void fold(float* p, int q) {
  if constexpr (M >= 1) {
    if constexpr (CNT > 1) {
      constexpr int half = CNT / 2;
      if constexpr (M >= 16) {
#pragma unroll
        for (int i = 0; i < half; ++i) p[i] = swap_sum<M>(p[i], p[i + half]);
      } else {
        const bool up = (q & M) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
          const float send = up ? p[i] : p[i + half];
          const float keep = up ? p[i + half] : p[i];
          p[i] = keep + lane_partner<M>(send);
        }
      }
      fold<half, M / 2>(p, q);
    } else {
      if constexpr (M >= 16) p[0] = swap_sum<M>(p[0], p[0]);
      else p[0] += lane_partner<M>(p[0]);
      fold<1, M / 2>(p, q);
    }
  }
}

template <int J, int G>
__global__ __launch_bounds__(kProjThreads) void logits_proj_fwd_kernel(ProjArgs a) {
  constexpr int H = J / 2, per = G / J, R = kRowsInFlight;
  static_assert(G >= J && G <= CXG_WAVE, "a group holds at least one lane per value");
  const int q = threadIdx.x % G, ro = threadIdx.x / G;
  const bool active = q < a.slots;
  float4 mv[J];
#pragma unroll
  for (int j = 0; j < J; ++j) mv[j] = active ? ld4(a.m + (int64_t)j * a.in + q * 4) : vzero<4>();
  const int64_t stride = kProjThreads / G;
  const int64_t begin = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t end = (begin + a.rows_per_block) < a.n_src ? (begin + a.rows_per_block) : a.n_src;
  const float* xq = a.x + q * 4;
  float4 cur[R];
#pragma unroll
  for (int u = 0; u < R; ++u) {
    const int64_t n = begin + ro + u * stride;
    cur[u] = (active && n < end) ? ld4(xq + n * a.ldx) : vzero<4>();
  }
  for (int64_t n0 = begin + ro; n0 < end; n0 += R * stride) {
    float4 nxt[R];                                  // the next step's rows load while this step's fold
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int64_t n = n0 + (R + u) * stride;
      nxt[u] = (active && n < end) ? ld4(xq + n * a.ldx) : vzero<4>();
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int64_t n = n0 + u * stride;
      float p[J];
#pragma unroll
      for (int j = 0; j < J; ++j) p[j] = vdot(cur[u], mv[j]);
      fold<J, G / 2>(p, q);
      const int j = q / per;
      if (q % per == 0 && n < end) {
        if (j < H) a.out_src[n * H + j] = p[0];
        else if (n < a.n_dst) a.out_dst[n * H + (j - H)] = p[0];
      }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) cur[u] = nxt[u];
  }
}

// H floats at p (zeros when !ok); 16-byte loads when H is a multiple of 4.
template <int H>
__device__ __forceinline__ void load_heads(const float* p, bool ok, float* dst) {
  if constexpr (H % 4 == 0) {
#pragma unroll
    for (int i = 0; i < H / 4; ++i) {
      const float4 v = ok ? ld4(p + 4 * i) : vzero<4>();
      dst[4 * i] = v.x; dst[4 * i + 1] = v.y; dst[4 * i + 2] = v.z; dst[4 * i + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < H; ++i) dst[i] = ok ? p[i] : 0.f;
  }
}

// grad_x[n, :] (+)= sum_j g[n, j] m[j, :]   (GX)      g[n, :] = (g_src[n, :], g_dst[n, :] or 0)
// partial[block, j, :] = sum over the block's rows of g[n, j] x[n, :]
template <int J, bool GX, bool ACC>
__global__ __launch_bounds__(kProjThreads) void logits_proj_bwd_kernel(ProjArgs a) {
  constexpr int H = J / 2;
  constexpr int R = J >= 16 ? 2 : kRowsInFlight;
  __shared__ float4 s_part[kProjThreads];
  const int q = threadIdx.x % a.group, ro = threadIdx.x / a.group;
  const bool active = q < a.slots;
  float4 mv[GX ? J : 1], acc[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    if (GX) mv[GX ? j : 0] = active ? ld4(a.m + (int64_t)j * a.in + q * 4) : vzero<4>();
    acc[j] = vzero<4>();
  }
  const int64_t stride = a.rpb;
  const int64_t begin = (int64_t)blockIdx.x * a.rows_per_block;
  const int64_t end = (begin + a.rows_per_block) < a.n_src ? (begin + a.rows_per_block) : a.n_src;
  for (int64_t n0 = begin + ro; n0 < end; n0 += R * stride) {
    float4 xv[R], old[(GX && ACC) ? R : 1];
    float g[R][J];
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int64_t n = n0 + u * stride;
      const bool in = n < end;
      xv[u] = (active && in) ? ld4(a.x + n * a.ldx + q * 4) : vzero<4>();
      if (GX && ACC) old[u] = (active && in) ? ld4(a.grad_x + n * a.ldg + q * 4) : vzero<4>();
      load_heads<H>(a.g_src + n * H, in, &g[u][0]);
      load_heads<H>(a.g_dst + n * H, in && n < a.n_dst, &g[u][H]);
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int64_t n = n0 + u * stride;
      if (GX) {
        float4 gx = (GX && ACC) ? old[(GX && ACC) ? u : 0] : vzero<4>();
#pragma unroll
        for (int j = 0; j < J; ++j) fma_into(gx, g[u][j], mv[GX ? j : 0]);
        if (active && n < end) *reinterpret_cast<float4*>(a.grad_x + n * a.ldg + q * 4) = gx;
      }
#pragma unroll
      for (int j = 0; j < J; ++j) fma_into(acc[j], g[u][j], xv[u]);
    }
  }
  float* row = a.partial + (int64_t)blockIdx.x * J * a.in;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    s_part[threadIdx.x] = acc[j];
    __syncthreads();
    if (ro == 0 && active) {
      float4 t = s_part[q];
      for (int r = 1; r < a.rpb; ++r) fma_into(t, 1.f, s_part[r * a.group + q]);
      *reinterpret_cast<float4*>(row + (int64_t)j * a.in + q * 4) = t;
    }
    __syncthreads();
  }
}

// out_src[c] / out_dst[c] = sum over blocks of the partial rows in a fixed order: the
// rows are cut into kReduceSlices contiguous runs, one thread sums a run (four
// interleaved chains) and the runs are added in run order.
constexpr int kReduceSlices = 16;

__global__ __launch_bounds__(64 * kReduceSlices) void att_partial_reduce_kernel(
    const float* __restrict__ partial, int blocks, int F, float* __restrict__ out_src,
    float* __restrict__ out_dst) {
  __shared__ float s_run[kReduceSlices][64];
  const int el = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + el;
  const int per = (blocks + kReduceSlices - 1) / kReduceSlices;
  const int b0 = sl * per, b1 = (b0 + per) < blocks ? (b0 + per) : blocks;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (c < 2 * F) {
    int b = b0;
    for (; b + 4 <= b1; b += 4) {
      s0 += partial[(int64_t)(b + 0) * 2 * F + c];
      s1 += partial[(int64_t)(b + 1) * 2 * F + c];
      s2 += partial[(int64_t)(b + 2) * 2 * F + c];
      s3 += partial[(int64_t)(b + 3) * 2 * F + c];
    }
    for (; b < b1; ++b) s0 += partial[(int64_t)b * 2 * F + c];
  }
  s_run[sl][el] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (sl == 0 && c < 2 * F) {
    float s = s_run[0][el];
#pragma unroll
    for (int q = 1; q < kReduceSlices; ++q) s += s_run[q][el];
    if (c < F) out_src[c] = s;
    else out_dst[c - F] = s;
  }
}

bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

// Block shape for S slots: rows per block step, contiguous rows per block, block count.
void block_shape(int slots, int64_t n_rows, AttArgs* a, int* blocks) {
  int r = kTargetThreads / slots;
  if (r < 1) r = 1;
  a->rpb = r;
  int64_t per = ceil_div(n_rows, kMaxBlocks);
  per = ceil_div(per > 0 ? per : 1, r) * r;
  a->rows_per_block = per;
  int64_t b = ceil_div(n_rows, per);
  if (b < 1) b = 1;
  *blocks = (int)b;
}

int bwd_vec(const AttArgs& a) {
  const int F = a.heads * a.channels;
  const uintptr_t bits = (uintptr_t)a.x | (uintptr_t)a.att_src | (uintptr_t)a.att_dst | (uintptr_t)a.grad_x;
  if (a.channels % 4 == 0 && (bits & 15) == 0 && F / 4 <= kMaxThreads) return 4;
  if (F <= kMaxThreads) return 1;
  return 0;
}

int check_shape(int64_t n_src, int64_t n_dst, int heads, int channels) {
  CXG_REQUIRE(n_src >= 0 && n_dst >= 0 && n_dst <= n_src, CXG_ERR_ARG,
              "need 0 <= n_dst <= n_src (got %lld, %lld)", (long long)n_dst, (long long)n_src);
  CXG_REQUIRE(heads >= 1 && channels >= 1, CXG_ERR_ARG, "heads/channels must be >= 1");
  CXG_REQUIRE((int64_t)heads * channels <= 4 * kMaxThreads, CXG_ERR_UNSUPPORTED,
              "heads*channels above %d", 4 * kMaxThreads);
  return CXG_OK;
}

int pow2_ceil(int x) { int p = 1; while (p < x) p <<= 1; return p; }

// Shapes the kernels that read the layer's input take: 4 | in <= 256, H in {1, 2, 4, 8}.
bool proj_shape_ok(int in, int heads) {
  return in >= 4 && in % 4 == 0 && in <= 4 * CXG_WAVE && (heads == 1 || heads == 2 || heads == 4 || heads == 8);
}

int proj_prepare(const float* x, int64_t ldx, const float* m, int64_t n_src, int64_t n_dst, int in,
                 int heads, ProjArgs* a, int* blocks) {
  CXG_REQUIRE(n_src >= 0 && n_dst >= 0 && n_dst <= n_src, CXG_ERR_ARG,
              "need 0 <= n_dst <= n_src (got %lld, %lld)", (long long)n_dst, (long long)n_src);
  CXG_REQUIRE(proj_shape_ok(in, heads), CXG_ERR_UNSUPPORTED,
              "in = %d, heads = %d: needs 4 | in <= %d and 1, 2, 4 or 8 heads", in, heads, 4 * CXG_WAVE);
  CXG_REQUIRE(ldx >= in && ldx % 4 == 0, CXG_ERR_ARG, "row stride %lld must be a multiple of 4 and >= in = %d",
              (long long)ldx, in);
  CXG_REQUIRE(m && (x || n_src == 0), CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE((((uintptr_t)x | (uintptr_t)m) & 15) == 0, CXG_ERR_ARG, "x and m must be 16-byte aligned");
  a->x = x; a->ldx = ldx; a->m = m; a->n_src = n_src; a->n_dst = n_dst; a->in = in;
  a->slots = in / 4;
  a->group = pow2_ceil(a->slots > 2 * heads ? a->slots : 2 * heads);
  a->rpb = kProjThreads / a->group;
  int64_t per = ceil_div(n_src > 0 ? n_src : 1, kMaxBlocks);
  per = ceil_div(per, a->rpb) * a->rpb;
  a->rows_per_block = per;
  const int64_t b = ceil_div(n_src, per);
  *blocks = b < 1 ? 1 : (int)b;
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

int cxg_attention_logits_fwd_f32(const float* x, const float* att_src, const float* att_dst,
                                 int64_t n_src, int64_t n_dst, int heads, int channels,
                                 float* out_src, float* out_dst, void* stream) {
  int rc = cxg::check_shape(n_src, n_dst, heads, channels);
  if (rc) return rc;
  if (n_src == 0) return CXG_OK;
  CXG_REQUIRE(x && att_src && att_dst && out_src && (out_dst || n_dst == 0), CXG_ERR_ARG, "null pointer");
  cxg::AttArgs a{};
  a.x = x; a.att_src = att_src; a.att_dst = att_dst; a.out_src = out_src; a.out_dst = out_dst;
  a.n_src = n_src; a.n_dst = n_dst; a.heads = heads; a.channels = channels;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int F = heads * channels;
  const uintptr_t bits = (uintptr_t)x | (uintptr_t)att_src | (uintptr_t)att_dst;
  int v = 0;
  for (int cand = 4; cand >= 1; cand >>= 1) {
    if (channels % cand != 0 || (bits & (uintptr_t)(4 * cand - 1)) != 0) continue;
    const int g = channels / cand;
    if (cxg::is_pow2(g) && g <= CXG_WAVE && F / cand <= cxg::kMaxThreads) { v = cand; break; }
  }
  if (v == 0) {
    const int64_t units = n_src * heads;
    hipLaunchKernelGGL(cxg::att_logits_fwd_generic_kernel, dim3((unsigned)cxg::ceil_div(units, 256)),
                       dim3(256), 0, st, a);
  } else {
    a.slots = F / v;
    int blocks = 1;
    cxg::block_shape(a.slots, n_src, &a, &blocks);
    const dim3 grid(blocks), block(a.slots * a.rpb);
    if (v == 4) hipLaunchKernelGGL(cxg::att_logits_fwd_kernel<4>, grid, block, 0, st, a);
    else if (v == 2) hipLaunchKernelGGL(cxg::att_logits_fwd_kernel<2>, grid, block, 0, st, a);
    else hipLaunchKernelGGL(cxg::att_logits_fwd_kernel<1>, grid, block, 0, st, a);
  }
  CXG_LAUNCH_CHECK("att_logits_fwd kernel");
  return CXG_OK;
}

size_t cxg_attention_logits_workspace_bytes(int64_t n_src, int heads, int channels) {
  if (n_src < 0 || heads < 1 || channels < 1) return 0;
  return (size_t)cxg::kMaxBlocks * 2 * (size_t)heads * (size_t)channels * sizeof(float) + 256;
}

int cxg_attention_logits_bwd_f32(const float* x, const float* att_src, const float* att_dst,
                                 const float* g_src, const float* g_dst, int64_t n_src, int64_t n_dst,
                                 int heads, int channels, float* grad_x, int accumulate,
                                 float* grad_att_src, float* grad_att_dst, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  int rc = cxg::check_shape(n_src, n_dst, heads, channels);
  if (rc) return rc;
  CXG_REQUIRE(att_src && att_dst && grad_att_src && grad_att_dst, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(n_src == 0 || (x && g_src && grad_x && (g_dst || n_dst == 0)), CXG_ERR_ARG, "null pointer");
  const size_t need = cxg_attention_logits_workspace_bytes(n_src, heads, channels);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  cxg::AttArgs a{};
  a.x = x; a.att_src = att_src; a.att_dst = att_dst; a.g_src = g_src; a.g_dst = g_dst;
  a.grad_x = grad_x; a.partial = reinterpret_cast<float*>(workspace);
  a.n_src = n_src; a.n_dst = n_dst; a.heads = heads; a.channels = channels;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int F = heads * channels;
  const int v = cxg::bwd_vec(a);
  CXG_REQUIRE(v != 0, CXG_ERR_UNSUPPORTED, "heads*channels = %d needs channels %% 4 == 0 and 16-byte "
              "aligned tensors above %d", F, cxg::kMaxThreads);
  a.slots = F / v;
  int blocks = 1;
  cxg::block_shape(a.slots, n_src, &a, &blocks);
  const dim3 grid(blocks), block(a.slots * a.rpb);
  const size_t lds = (size_t)2 * block.x * v * sizeof(float);
  if (v == 4 && accumulate) hipLaunchKernelGGL((cxg::att_logits_bwd_kernel<4, true>), grid, block, lds, st, a);
  else if (v == 4) hipLaunchKernelGGL((cxg::att_logits_bwd_kernel<4, false>), grid, block, lds, st, a);
  else if (accumulate) hipLaunchKernelGGL((cxg::att_logits_bwd_kernel<1, true>), grid, block, lds, st, a);
  else hipLaunchKernelGGL((cxg::att_logits_bwd_kernel<1, false>), grid, block, lds, st, a);
  CXG_LAUNCH_CHECK("att_logits_bwd_kernel");
  hipLaunchKernelGGL(cxg::att_partial_reduce_kernel, dim3((unsigned)cxg::ceil_div(2 * F, 64)),
                     dim3(64 * cxg::kReduceSlices), 0,
                     st, a.partial, blocks, F, grad_att_src, grad_att_dst);
  CXG_LAUNCH_CHECK("att_partial_reduce_kernel");
  return CXG_OK;
}

int cxg_attention_logits_proj_supported(int in, int heads) { return cxg::proj_shape_ok(in, heads) ? 1 : 0; }

int cxg_attention_logits_proj_fwd_f32(const float* x, int64_t ldx, const float* m, int64_t n_src,
                                      int64_t n_dst, int in, int heads, float* out_src, float* out_dst,
                                      void* stream) {
  cxg::ProjArgs a{};
  int blocks = 1;
  int rc = cxg::proj_prepare(x, ldx, m, n_src, n_dst, in, heads, &a, &blocks);
  if (rc) return rc;
  if (n_src == 0) return CXG_OK;
  CXG_REQUIRE(out_src && (out_dst || n_dst == 0), CXG_ERR_ARG, "null pointer");
  a.out_src = out_src; a.out_dst = out_dst;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(blocks), block(cxg::kProjThreads);
#define CXG_PROJ_FWD(JV, GV)                                                                          \
  if (2 * heads == JV && a.group == GV) {                                                             \
    if constexpr (GV >= JV) hipLaunchKernelGGL((cxg::logits_proj_fwd_kernel<JV, GV>), grid, block, 0, st, a); \
  }
#define CXG_PROJ_FWD_G(GV) CXG_PROJ_FWD(2, GV) CXG_PROJ_FWD(4, GV) CXG_PROJ_FWD(8, GV) CXG_PROJ_FWD(16, GV)
  CXG_PROJ_FWD_G(2) CXG_PROJ_FWD_G(4) CXG_PROJ_FWD_G(8) CXG_PROJ_FWD_G(16) CXG_PROJ_FWD_G(32) CXG_PROJ_FWD_G(64)
#undef CXG_PROJ_FWD_G
#undef CXG_PROJ_FWD
  CXG_LAUNCH_CHECK("logits_proj_fwd_kernel");
  return CXG_OK;
}

size_t cxg_attention_logits_proj_workspace_bytes(int in, int heads) {
  if (in < 1 || heads < 1) return 0;
  return (size_t)cxg::kMaxBlocks * 2 * (size_t)heads * (size_t)in * sizeof(float) + 256;
}

int cxg_attention_logits_proj_bwd_f32(const float* x, int64_t ldx, const float* m, const float* g_src,
                                      const float* g_dst, int64_t n_src, int64_t n_dst, int in, int heads,
                                      float* grad_x, int64_t ldg, int accumulate, float* grad_m,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  cxg::ProjArgs a{};
  int blocks = 1;
  int rc = cxg::proj_prepare(x, ldx, m, n_src, n_dst, in, heads, &a, &blocks);
  if (rc) return rc;
  CXG_REQUIRE(grad_m, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(n_src == 0 || (g_src && (g_dst || n_dst == 0)), CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(heads % 4 != 0 || (((uintptr_t)g_src | (uintptr_t)g_dst) & 15) == 0, CXG_ERR_ARG,
              "g_src and g_dst must be 16-byte aligned");
  CXG_REQUIRE(!grad_x || (ldg >= in && ldg % 4 == 0 && ((uintptr_t)grad_x & 15) == 0), CXG_ERR_ARG,
              "grad_x must be 16-byte aligned with a row stride that is a multiple of 4 and >= in");
  const size_t need = cxg_attention_logits_proj_workspace_bytes(in, heads);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  a.g_src = g_src; a.g_dst = g_dst ? g_dst : g_src; a.grad_x = grad_x; a.ldg = ldg;
  a.partial = reinterpret_cast<float*>(workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid(blocks), block(cxg::kProjThreads);
  const int mode = !grad_x ? 0 : (accumulate ? 2 : 1);
#define CXG_PROJ_BWD(JV)                                                                              \
  do {                                                                                                \
    if (mode == 0) hipLaunchKernelGGL((cxg::logits_proj_bwd_kernel<JV, false, false>), grid, block, 0, st, a); \
    else if (mode == 1) hipLaunchKernelGGL((cxg::logits_proj_bwd_kernel<JV, true, false>), grid, block, 0, st, a); \
    else hipLaunchKernelGGL((cxg::logits_proj_bwd_kernel<JV, true, true>), grid, block, 0, st, a);    \
  } while (0)
  switch (heads) {
    case 1: CXG_PROJ_BWD(2); break;
    case 2: CXG_PROJ_BWD(4); break;
    case 4: CXG_PROJ_BWD(8); break;
    default: CXG_PROJ_BWD(16); break;
  }
#undef CXG_PROJ_BWD
  CXG_LAUNCH_CHECK("logits_proj_bwd_kernel");
  const int F = heads * in;                      // grad_m is 2 * F floats
  hipLaunchKernelGGL(cxg::att_partial_reduce_kernel, dim3((unsigned)cxg::ceil_div(2 * F, 64)),
                     dim3(64 * cxg::kReduceSlices), 0, st, a.partial, blocks, F, grad_m, grad_m + F);
  CXG_LAUNCH_CHECK("att_partial_reduce_kernel");
  return CXG_OK;
}

}  // extern "C"
