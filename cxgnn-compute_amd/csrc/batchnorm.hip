// Batch normalisation over the rows of a node-feature matrix x[n, c] (the layer between
// the convolutions of the upstream models, torch.nn.BatchNorm1d in cxgnncomp/model.py:28):
//   statistics  mean[c], biased variance -> invstd[c] = 1/sqrt(var + eps), unbiased variance
//   apply       y = (x - mean) * invstd * gamma + beta            (optionally max(., 0))
//   backward    dbeta = sum dy, dgamma = sum dy * xhat,
//               dx = gamma * invstd * (dy - dbeta/n - xhat * dgamma/n),  xhat = (x - mean) * invstd
//               (with the fused max(., 0): dy counts only where y > 0, y recomputed from x)
//
// Layout: a row is cut into c/V slots of V floats (V = 4 where the shape allows).  A block
// of 256 threads is TX slots wide and TY = 256/TX rows deep and owns a contiguous run of
// rows; thread (tx, ty) keeps its slot and visits rows ty, ty + TY, ...: a wave reads whole
// consecutive rows, and per-column state stays in registers.  Column statistics are
// Welford means / sums of squared deviations of x - x[0, :] per thread (shifted by the
// first row, so that a column mean far from zero costs no accuracy), merged pairwise (Chan) over the
// TY row offsets in LDS, written as one partial row per block and merged again, in block
// order, by a second kernel (one wave per column).  Grid sizes depend on the shape only,
// so results are reproducible bit for bit.  The same layout serves the plain column sum
// (the bias gradient of a linear layer, g.sum(0)).
#include "cxg_common.hpp"

namespace cxg {
namespace {

constexpr int kBnThreads = 256;
constexpr int kBnMaxRowBlocks = 1024;
constexpr int kBnRowsPerThread = 16;        // target rows per thread of the reductions

struct BnGeom {
  int v;             // floats per slot
  int tx_shift;      // TX = 1 << tx_shift slots per block row
  int col_tiles;     // grid.y
  int row_blocks;    // grid.x
  int64_t rows_per_block;
};

BnGeom bn_geometry(int64_t n, int c, bool vec4) {
  BnGeom g;
  g.v = vec4 ? 4 : 1;
  const int slots = c / g.v;
  g.tx_shift = 0;
  while ((1 << g.tx_shift) < slots && (1 << g.tx_shift) < kBnThreads) ++g.tx_shift;
  const int tx = 1 << g.tx_shift, ty = kBnThreads / tx;
  g.col_tiles = (slots + tx - 1) / tx;
  int64_t rb = ceil_div(n, (int64_t)ty * kBnRowsPerThread);
  if (rb > kBnMaxRowBlocks) rb = kBnMaxRowBlocks;
  if (rb < 1) rb = 1;
  g.rows_per_block = ceil_div(n, rb);
  g.row_blocks = (int)ceil_div(n, g.rows_per_block);
  if (g.row_blocks < 1) g.row_blocks = 1;
  return g;
}

template <int V> __device__ __forceinline__ void load_v(const float* __restrict__ p, float (&v)[V]) {
  if constexpr (V == 4) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    v[0] = p[0];
  }
}
template <int V> __device__ __forceinline__ void store_v(float* __restrict__ p, const float (&v)[V]) {
  if constexpr (V == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  else p[0] = v[0];
}

// (count, mean, m2) of a set <- union with a second, disjoint set
__device__ __forceinline__ void chan_merge(float& na, float& ma, float& qa, float nb, float mb, float qb) {
  if (nb == 0.f) return;
  const float n = na + nb, d = mb - ma, f = nb / n;
  ma += d * f;
  qa += qb + d * d * na * f;
  na = n;
}

struct BnBlock {
  int tx_i, ty_i, ty, slot;
  bool live;
  int64_t r_begin, r_end;
  __device__ __forceinline__ BnBlock(int64_t n, int c, int v, int tx_shift, int64_t rows_per_block) {
    const int tx = 1 << tx_shift;
    tx_i = threadIdx.x & (tx - 1);
    ty_i = threadIdx.x >> tx_shift;
    ty = kBnThreads >> tx_shift;
    slot = blockIdx.y * tx + tx_i;
    live = slot < c / v;
    r_begin = (int64_t)blockIdx.x * rows_per_block;
    r_end = r_begin + rows_per_block < n ? r_begin + rows_per_block : n;
  }
};

// partial[b][0][col] = mean, partial[b][1][col] = m2 of x - x[0, col] over the rows of block b
template <int V>
__global__ __launch_bounds__(kBnThreads) void bn_stats_partial_kernel(
    const float* __restrict__ x, int64_t n, int c, int64_t ldx, int tx_shift, int64_t rows_per_block,
    float* __restrict__ partial) {
  __shared__ float s_mean[kBnThreads * V], s_m2[kBnThreads * V], s_cnt[kBnThreads];
  const BnBlock b(n, c, V, tx_shift, rows_per_block);
  float mean[V], m2[V], cnt = 0.f;
#pragma unroll
  for (int i = 0; i < V; ++i) { mean[i] = 0.f; m2[i] = 0.f; }
  if (b.live) {
    float k[V];
    load_v<V>(x + (int64_t)b.slot * V, k);
    for (int64_t r = b.r_begin + b.ty_i; r < b.r_end; r += b.ty) {
      float v[V];
      load_v<V>(x + r * ldx + (int64_t)b.slot * V, v);
      cnt += 1.f;
      const float inv = 1.0f / cnt;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        v[i] -= k[i];
        const float d = v[i] - mean[i];
        mean[i] += d * inv;
        m2[i] += d * (v[i] - mean[i]);
      }
    }
  }
  s_cnt[threadIdx.x] = cnt;
#pragma unroll
  for (int i = 0; i < V; ++i) { s_mean[threadIdx.x * V + i] = mean[i]; s_m2[threadIdx.x * V + i] = m2[i]; }
  __syncthreads();
  if (b.ty_i == 0 && b.live) {
    const int tx = 1 << tx_shift;
    for (int j = 1; j < b.ty; ++j) {
      const int t = j * tx + b.tx_i;
      const float nb = s_cnt[t];
#pragma unroll
      for (int i = 0; i < V; ++i) {
        float na = cnt;                       // the count is shared by the V columns: merge each from the same na
        chan_merge(na, mean[i], m2[i], nb, s_mean[t * V + i], s_m2[t * V + i]);
      }
      cnt += nb;
    }
    float* out = partial + (size_t)blockIdx.x * 2 * c + (size_t)b.slot * V;
    store_v<V>(out, mean);
    store_v<V>(out + c, m2);
  }
}

// One wave per column: merge the per-block partials in block order.
__global__ __launch_bounds__(kBnThreads) void bn_stats_final_kernel(
    const float* __restrict__ partial, const float* __restrict__ x, int row_blocks, int64_t rows_per_block,
    int64_t n, int c, float eps, float* __restrict__ mean_out, float* __restrict__ invstd_out, float* __restrict__ var_unbiased_out) {
  const int lane = lane_id();
  const int col = blockIdx.x * (kBnThreads / CXG_WAVE) + (threadIdx.x >> 6);
  if (col >= c) return;
  auto rows_of = [&](int b) -> float {
    const int64_t r0 = (int64_t)b * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < n ? r0 + rows_per_block : n;
    return (float)(r1 - r0);
  };
  // lane l takes the contiguous run of blocks [l*per, (l+1)*per)
  const int per = (row_blocks + CXG_WAVE - 1) / CXG_WAVE;
  float cnt = 0.f, mean = 0.f, m2 = 0.f;
  for (int b = lane * per; b < (lane + 1) * per && b < row_blocks; ++b)
    chan_merge(cnt, mean, m2, rows_of(b), partial[(size_t)b * 2 * c + col], partial[(size_t)b * 2 * c + c + col]);
  // neighbouring runs pairwise: after step s lane l (l % 2s == 0) holds runs l .. l+2s-1
  for (int s = 1; s < CXG_WAVE; s <<= 1) {
    const float nb = __shfl_down(cnt, s, CXG_WAVE), mb = __shfl_down(mean, s, CXG_WAVE),
                qb = __shfl_down(m2, s, CXG_WAVE);
    if ((lane & (2 * s - 1)) == 0) chan_merge(cnt, mean, m2, nb, mb, qb);
  }
  if (lane == 0) {
    const float var = m2 / (float)n;
    mean_out[col] = x[col] + mean;
    invstd_out[col] = 1.0f / sqrtf(var + eps);
    if (var_unbiased_out) var_unbiased_out[col] = n > 1 ? m2 / (float)(n - 1) : var;
  }
}

template <int V, bool RELU>
__global__ __launch_bounds__(kBnThreads) void bn_apply_kernel(
    const float* __restrict__ x, int64_t n, int c, int64_t ldx, int tx_shift, int64_t rows_per_block,
    const float* __restrict__ mean, const float* __restrict__ invstd, const float* __restrict__ gamma,
    const float* __restrict__ beta, float* __restrict__ y, int64_t ldy) {
  const BnBlock b(n, c, V, tx_shift, rows_per_block);
  if (!b.live) return;
  float mu[V], sc[V], sh[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int col = b.slot * V + i;
    mu[i] = mean[col];
    sc[i] = invstd[col] * (gamma ? gamma[col] : 1.0f);
    sh[i] = beta ? beta[col] : 0.0f;
  }
  for (int64_t r = b.r_begin + b.ty_i; r < b.r_end; r += b.ty) {
    float v[V];
    load_v<V>(x + r * ldx + (int64_t)b.slot * V, v);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      v[i] = (v[i] - mu[i]) * sc[i] + sh[i];
      if (RELU) v[i] = fmaxf(v[i], 0.f);
    }
    store_v<V>(y + r * ldy + (int64_t)b.slot * V, v);
  }
}

// partial[b][0][col] = sum dy, partial[b][1][col] = sum dy * xhat over the rows of block b
template <int V, bool RELU>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_partial_kernel(
    const float* __restrict__ x, const float* __restrict__ dy, int64_t n, int c, int64_t ldx, int64_t lddy,
    int tx_shift, int64_t rows_per_block, const float* __restrict__ mean, const float* __restrict__ invstd,
    const float* __restrict__ gamma, const float* __restrict__ beta, float* __restrict__ partial) {
  __shared__ float s_a[kBnThreads * V], s_b[kBnThreads * V];
  const BnBlock b(n, c, V, tx_shift, rows_per_block);
  float sa[V], sb[V], mu[V], is[V], sc[V], sh[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    sa[i] = 0.f; sb[i] = 0.f;
    const int col = b.slot * V + i;
    mu[i] = b.live ? mean[col] : 0.f;
    is[i] = b.live ? invstd[col] : 0.f;
    sc[i] = is[i] * ((b.live && gamma) ? gamma[col] : 1.0f);
    sh[i] = (b.live && beta) ? beta[col] : 0.0f;
  }
  if (b.live) {
    for (int64_t r = b.r_begin + b.ty_i; r < b.r_end; r += b.ty) {
      float v[V], g[V];
      load_v<V>(x + r * ldx + (int64_t)b.slot * V, v);
      load_v<V>(dy + r * lddy + (int64_t)b.slot * V, g);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = v[i] - mu[i];
        if (RELU && !(d * sc[i] + sh[i] > 0.f)) g[i] = 0.f;
        sa[i] += g[i];
        sb[i] += g[i] * (d * is[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < V; ++i) { s_a[threadIdx.x * V + i] = sa[i]; s_b[threadIdx.x * V + i] = sb[i]; }
  __syncthreads();
  if (b.ty_i == 0 && b.live) {
    const int tx = 1 << tx_shift;
    for (int j = 1; j < b.ty; ++j) {
      const int t = j * tx + b.tx_i;
#pragma unroll
      for (int i = 0; i < V; ++i) { sa[i] += s_a[t * V + i]; sb[i] += s_b[t * V + i]; }
    }
    float* out = partial + (size_t)blockIdx.x * 2 * c + (size_t)b.slot * V;
    store_v<V>(out, sa);
    store_v<V>(out + c, sb);
  }
}

__global__ __launch_bounds__(kBnThreads) void bn_bwd_final_kernel(
    const float* __restrict__ partial, int row_blocks, int c, float* __restrict__ dgamma,
    float* __restrict__ dbeta) {
  const int lane = lane_id();
  const int col = blockIdx.x * (kBnThreads / CXG_WAVE) + (threadIdx.x >> 6);
  if (col >= c) return;
  const int per = (row_blocks + CXG_WAVE - 1) / CXG_WAVE;
  float a = 0.f, q = 0.f;
  for (int b = lane * per; b < (lane + 1) * per && b < row_blocks; ++b) {
    a += partial[(size_t)b * 2 * c + col];
    q += partial[(size_t)b * 2 * c + c + col];
  }
  for (int s = 1; s < CXG_WAVE; s <<= 1) {
    const float a2 = __shfl_down(a, s, CXG_WAVE), q2 = __shfl_down(q, s, CXG_WAVE);
    if ((lane & (2 * s - 1)) == 0) { a += a2; q += q2; }
  }
  if (lane == 0) { dbeta[col] = a; dgamma[col] = q; }
}

template <int V, bool RELU>
__global__ __launch_bounds__(kBnThreads) void bn_bwd_dx_kernel(
    const float* __restrict__ x, const float* __restrict__ dy, int64_t n, int c, int64_t ldx, int64_t lddy,
    int tx_shift, int64_t rows_per_block, const float* __restrict__ mean, const float* __restrict__ invstd,
    const float* __restrict__ gamma, const float* __restrict__ beta, const float* __restrict__ dgamma,
    const float* __restrict__ dbeta, float* __restrict__ dx, int64_t lddx) {
  const BnBlock b(n, c, V, tx_shift, rows_per_block);
  if (!b.live) return;
  const float inv_n = 1.0f / (float)n;
  float mu[V], is[V], sc[V], sh[V], ma[V], mq[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    const int col = b.slot * V + i;
    mu[i] = mean[col];
    is[i] = invstd[col];
    sc[i] = is[i] * (gamma ? gamma[col] : 1.0f);
    sh[i] = beta ? beta[col] : 0.0f;
    ma[i] = dbeta[col] * inv_n;
    mq[i] = dgamma[col] * inv_n;
  }
  for (int64_t r = b.r_begin + b.ty_i; r < b.r_end; r += b.ty) {
    float v[V], g[V];
    load_v<V>(x + r * ldx + (int64_t)b.slot * V, v);
    load_v<V>(dy + r * lddy + (int64_t)b.slot * V, g);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float d = v[i] - mu[i];
      if (RELU && !(d * sc[i] + sh[i] > 0.f)) g[i] = 0.f;
      v[i] = sc[i] * (g[i] - ma[i] - d * is[i] * mq[i]);
    }
    store_v<V>(dx + r * lddx + (int64_t)b.slot * V, v);
  }
}

// partial[b][col] = sum of x[r, col] over the rows of block b (the bias gradient of a linear layer)
template <int V>
__global__ __launch_bounds__(kBnThreads) void column_sum_partial_kernel(
    const float* __restrict__ x, int64_t n, int c, int64_t ldx, int tx_shift, int64_t rows_per_block,
    float* __restrict__ partial) {
  __shared__ float s_a[kBnThreads * V];
  const BnBlock b(n, c, V, tx_shift, rows_per_block);
  float sa[V];
#pragma unroll
  for (int i = 0; i < V; ++i) sa[i] = 0.f;
  if (b.live) {
    for (int64_t r = b.r_begin + b.ty_i; r < b.r_end; r += b.ty) {
      float v[V];
      load_v<V>(x + r * ldx + (int64_t)b.slot * V, v);
#pragma unroll
      for (int i = 0; i < V; ++i) sa[i] += v[i];
    }
  }
#pragma unroll
  for (int i = 0; i < V; ++i) s_a[threadIdx.x * V + i] = sa[i];
  __syncthreads();
  if (b.ty_i == 0 && b.live) {
    const int tx = 1 << tx_shift;
    for (int j = 1; j < b.ty; ++j) {
      const int t = j * tx + b.tx_i;
#pragma unroll
      for (int i = 0; i < V; ++i) sa[i] += s_a[t * V + i];
    }
    store_v<V>(partial + (size_t)blockIdx.x * c + (size_t)b.slot * V, sa);
  }
}

__global__ __launch_bounds__(kBnThreads) void column_sum_final_kernel(
    const float* __restrict__ partial, int row_blocks, int c, float* __restrict__ out) {
  const int lane = lane_id();
  const int col = blockIdx.x * (kBnThreads / CXG_WAVE) + (threadIdx.x >> 6);
  if (col >= c) return;
  const int per = (row_blocks + CXG_WAVE - 1) / CXG_WAVE;
  float a = 0.f;
  for (int b = lane * per; b < (lane + 1) * per && b < row_blocks; ++b) a += partial[(size_t)b * c + col];
  for (int s = 1; s < CXG_WAVE; s <<= 1) {
    const float a2 = __shfl_down(a, s, CXG_WAVE);
    if ((lane & (2 * s - 1)) == 0) a += a2;
  }
  if (lane == 0) out[col] = a;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_batchnorm_workspace_bytes(int64_t n, int c) {
  if (n <= 0 || c <= 0) return 0;
  // the row-block count of the scalar layout is never below that of the vector layout
  const cxg::BnGeom g = cxg::bn_geometry(n, c, false);
  return (size_t)g.row_blocks * 2 * (size_t)c * sizeof(float);
}

int cxg_batchnorm_stats_f32(const float* x, int64_t n, int c, int64_t ldx, float eps, float* mean,
                            float* invstd, float* var_unbiased, void* workspace, size_t workspace_bytes,
                            void* stream) {
  CXG_REQUIRE(n >= 1 && c >= 1 && ldx >= c, CXG_ERR_ARG, "batchnorm_stats: bad n/c/ldx");
  CXG_REQUIRE(x && mean && invstd && workspace, CXG_ERR_ARG, "batchnorm_stats: null x/mean/invstd/workspace");
  CXG_REQUIRE(workspace_bytes >= cxg_batchnorm_workspace_bytes(n, c), CXG_ERR_ARG,
              "batchnorm_stats: workspace of %zu bytes, %zu needed", workspace_bytes,
              cxg_batchnorm_workspace_bytes(n, c));
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool v4 = c % 4 == 0 && ldx % 4 == 0 && cxg::aligned16(x);
  const cxg::BnGeom g = cxg::bn_geometry(n, c, v4);
  float* partial = static_cast<float*>(workspace);
  dim3 grid(g.row_blocks, g.col_tiles), block(cxg::kBnThreads);
  if (v4)
    hipLaunchKernelGGL(cxg::bn_stats_partial_kernel<4>, grid, block, 0, st, x, n, c, ldx, g.tx_shift,
                       g.rows_per_block, partial);
  else
    hipLaunchKernelGGL(cxg::bn_stats_partial_kernel<1>, grid, block, 0, st, x, n, c, ldx, g.tx_shift,
                       g.rows_per_block, partial);
  CXG_LAUNCH_CHECK("bn_stats_partial_kernel");
  const int waves = cxg::kBnThreads / CXG_WAVE;
  hipLaunchKernelGGL(cxg::bn_stats_final_kernel, dim3((c + waves - 1) / waves), block, 0, st, partial, x,
                     g.row_blocks, g.rows_per_block, n, c, eps, mean, invstd, var_unbiased);
  CXG_LAUNCH_CHECK("bn_stats_final_kernel");
  return CXG_OK;
}

int cxg_batchnorm_apply_f32(const float* x, int64_t n, int c, int64_t ldx, const float* mean,
                            const float* invstd, const float* gamma, const float* beta, float* y,
                            int64_t ldy, int relu, void* stream) {
  CXG_REQUIRE(n >= 0 && c >= 1 && ldx >= c && ldy >= c, CXG_ERR_ARG, "batchnorm_apply: bad n/c/ld");
  if (n == 0) return CXG_OK;
  CXG_REQUIRE(x && y && mean && invstd, CXG_ERR_ARG, "batchnorm_apply: null x/y/mean/invstd");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool v4 = c % 4 == 0 && ldx % 4 == 0 && ldy % 4 == 0 && cxg::aligned16(x) && cxg::aligned16(y);
  const cxg::BnGeom g = cxg::bn_geometry(n, c, v4);
  dim3 grid(g.row_blocks, g.col_tiles), block(cxg::kBnThreads);
#define CXG_BN_APPLY(VV, RR)                                                                       \
  hipLaunchKernelGGL((cxg::bn_apply_kernel<VV, RR>), grid, block, 0, st, x, n, c, ldx, g.tx_shift, \
                     g.rows_per_block, mean, invstd, gamma, beta, y, ldy)
  if (v4) { if (relu) CXG_BN_APPLY(4, true); else CXG_BN_APPLY(4, false); }
  else { if (relu) CXG_BN_APPLY(1, true); else CXG_BN_APPLY(1, false); }
#undef CXG_BN_APPLY
  CXG_LAUNCH_CHECK("bn_apply_kernel");
  return CXG_OK;
}

int cxg_batchnorm_bwd_f32(const float* x, const float* dy, int64_t n, int c, int64_t ldx, int64_t lddy,
                          const float* mean, const float* invstd, const float* gamma, const float* beta,
                          int relu, float* dx, int64_t lddx, float* dgamma, float* dbeta, void* workspace,
                          size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n >= 1 && c >= 1 && ldx >= c && lddy >= c && lddx >= c, CXG_ERR_ARG, "batchnorm_bwd: bad n/c/ld");
  CXG_REQUIRE(x && dy && mean && invstd && dx && dgamma && dbeta && workspace, CXG_ERR_ARG,
              "batchnorm_bwd: null pointer");
  CXG_REQUIRE(workspace_bytes >= cxg_batchnorm_workspace_bytes(n, c), CXG_ERR_ARG,
              "batchnorm_bwd: workspace of %zu bytes, %zu needed", workspace_bytes,
              cxg_batchnorm_workspace_bytes(n, c));
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool v4 = c % 4 == 0 && ldx % 4 == 0 && lddy % 4 == 0 && lddx % 4 == 0 && cxg::aligned16(x) &&
                  cxg::aligned16(dy) && cxg::aligned16(dx);
  const cxg::BnGeom g = cxg::bn_geometry(n, c, v4);
  float* partial = static_cast<float*>(workspace);
  dim3 grid(g.row_blocks, g.col_tiles), block(cxg::kBnThreads);
#define CXG_BN_PART(VV, RR)                                                                           \
  hipLaunchKernelGGL((cxg::bn_bwd_partial_kernel<VV, RR>), grid, block, 0, st, x, dy, n, c, ldx, lddy, \
                     g.tx_shift, g.rows_per_block, mean, invstd, gamma, beta, partial)
  if (v4) { if (relu) CXG_BN_PART(4, true); else CXG_BN_PART(4, false); }
  else { if (relu) CXG_BN_PART(1, true); else CXG_BN_PART(1, false); }
#undef CXG_BN_PART
  CXG_LAUNCH_CHECK("bn_bwd_partial_kernel");
  const int waves = cxg::kBnThreads / CXG_WAVE;
  hipLaunchKernelGGL(cxg::bn_bwd_final_kernel, dim3((c + waves - 1) / waves), block, 0, st, partial,
                     g.row_blocks, c, dgamma, dbeta);
  CXG_LAUNCH_CHECK("bn_bwd_final_kernel");
#define CXG_BN_DX(VV, RR)                                                                          \
  hipLaunchKernelGGL((cxg::bn_bwd_dx_kernel<VV, RR>), grid, block, 0, st, x, dy, n, c, ldx, lddy,   \
                     g.tx_shift, g.rows_per_block, mean, invstd, gamma, beta, dgamma, dbeta, dx, lddx)
  if (v4) { if (relu) CXG_BN_DX(4, true); else CXG_BN_DX(4, false); }
  else { if (relu) CXG_BN_DX(1, true); else CXG_BN_DX(1, false); }
#undef CXG_BN_DX
  CXG_LAUNCH_CHECK("bn_bwd_dx_kernel");
  return CXG_OK;
}

int cxg_column_sum_f32(const float* x, int64_t n, int c, int64_t ldx, float* out, void* workspace,
                       size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n >= 0 && c >= 1 && ldx >= c, CXG_ERR_ARG, "column_sum: bad n/c/ldx");
  CXG_REQUIRE(out, CXG_ERR_ARG, "column_sum: null out");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int waves = cxg::kBnThreads / CXG_WAVE;
  if (n == 0) {                                  // no rows: the merge of zero partial rows writes the zeros
    hipLaunchKernelGGL(cxg::column_sum_final_kernel, dim3((c + waves - 1) / waves), dim3(cxg::kBnThreads), 0, st,
                       static_cast<const float*>(nullptr), 0, c, out);
    CXG_LAUNCH_CHECK("column_sum_final_kernel");
    return CXG_OK;
  }
  CXG_REQUIRE(x && workspace, CXG_ERR_ARG, "column_sum: null x/workspace");
  CXG_REQUIRE(workspace_bytes >= cxg_batchnorm_workspace_bytes(n, c), CXG_ERR_ARG,
              "column_sum: workspace of %zu bytes, %zu needed", workspace_bytes,
              cxg_batchnorm_workspace_bytes(n, c));
  const bool v4 = c % 4 == 0 && ldx % 4 == 0 && cxg::aligned16(x);
  const cxg::BnGeom g = cxg::bn_geometry(n, c, v4);
  float* partial = static_cast<float*>(workspace);
  dim3 grid(g.row_blocks, g.col_tiles), block(cxg::kBnThreads);
  if (v4)
    hipLaunchKernelGGL(cxg::column_sum_partial_kernel<4>, grid, block, 0, st, x, n, c, ldx, g.tx_shift,
                       g.rows_per_block, partial);
  else
    hipLaunchKernelGGL(cxg::column_sum_partial_kernel<1>, grid, block, 0, st, x, n, c, ldx, g.tx_shift,
                       g.rows_per_block, partial);
  CXG_LAUNCH_CHECK("column_sum_partial_kernel");
  hipLaunchKernelGGL(cxg::column_sum_final_kernel, dim3((c + waves - 1) / waves), block, 0, st, partial,
                     g.row_blocks, c, out);
  CXG_LAUNCH_CHECK("column_sum_final_kernel");
  return CXG_OK;
}

}  // extern "C"
