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

}  // extern "C"
