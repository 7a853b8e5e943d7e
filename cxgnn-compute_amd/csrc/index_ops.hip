// Integer / index work on CSR graphs: transposition (the graph the backward
// pass gathers over), row-id expansion, 1/degree edge values and relation
// padding.  All results are bit-exact functions of their inputs.
#include "cxg_common.hpp"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

namespace cxg {
namespace {

constexpr int kBlock = 256;

// rows[k] = row containing edge position pos(k): the r with ptr[r] <= p < ptr[r+1].
__device__ __forceinline__ int64_t row_of_position(const int64_t* __restrict__ ptr, int64_t n_rows,
                                                   int64_t p) {
  // upper_bound(ptr[0..n_rows], p) - 1
  int64_t lo = 0, hi = n_rows + 1;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (ptr[mid] <= p) lo = mid + 1;
    else hi = mid;
  }
  return lo - 1;
}

__global__ void transpose_fill_kernel(const int64_t* __restrict__ ptr, int64_t n_rows,
                                      const int64_t* __restrict__ sorted_src,
                                      const int64_t* __restrict__ perm, int64_t n_edges,
                                      int64_t n_cols, int64_t* __restrict__ ptr_t,
                                      int64_t* __restrict__ idx_t) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k < n_edges) idx_t[k] = row_of_position(ptr, n_rows, perm[k]);
  if (k <= n_cols) {
    // ptr_t[c] = number of edges whose source is < c
    int64_t lo = 0, hi = n_edges;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (sorted_src[mid] < k) lo = mid + 1;
      else hi = mid;
    }
    ptr_t[k] = lo;
  }
}

// Narrow form of the transposition, for graphs whose row, column and edge counts all fit
// 32 bits: the sort moves 4-byte keys and one 8-byte value per edge that carries the
// edge's row next to its position, so no search by (random) position follows the sort.
struct ColumnKey {
  __host__ __device__ uint32_t operator()(int64_t v) const { return (uint32_t)v; }
};
using ColumnKeyIter = rocprim::transform_iterator<const int64_t*, ColumnKey, uint32_t>;

// Row of every edge position, written as int64 row ids (MODE 0) or packed with the
// position for the narrow transposition (MODE 1).  One wave walks kRowSpan positions.
constexpr int kRowSpan = 8 * CXG_WAVE;

template <int MODE>
__global__ __launch_bounds__(kBlock) void expand_rows_kernel(const int64_t* __restrict__ ptr,
                                                             int64_t n_rows, int64_t n_edges,
                                                             void* __restrict__ out) {
  const int lane = lane_id();
  const int64_t w = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
  const int64_t k0 = uniform_i64(w * kRowSpan);
  if (k0 >= n_edges) return;
  RowWalker walk;
  walk.init(ptr, n_rows, (MODE == 0 ? ptr[0] : 0) + k0);   // row ids count positions from ptr[0]
  for (int c = 0; c < kRowSpan; c += CXG_WAVE) {
    const int64_t k = k0 + c + lane;
    if (k0 + c >= n_edges) break;
    const int64_t row = walk.row_of(c + lane, k < n_edges);
    if (k < n_edges) {
      if (MODE == 0) reinterpret_cast<int64_t*>(out)[k] = row;
      else reinterpret_cast<uint64_t*>(out)[k] = ((uint64_t)row << 32) | (uint64_t)k;
    }
  }
}

// perm / idx_t from the sorted packed values (in place over `perm`); ptr_t[c] = number of
// edges whose source is < c, by a search of the sorted keys per column (one thread per
// column: the columns may outnumber the edges by far, e.g. a sampled layer over all nodes).
__global__ void transpose_unpack_kernel(const uint32_t* __restrict__ sorted_key, int64_t n_edges,
                                        int64_t n_cols, int64_t* __restrict__ perm,
                                        int64_t* __restrict__ idx_t, int64_t* __restrict__ ptr_t) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k < n_edges) {
    const uint64_t v = (uint64_t)perm[k];
    perm[k] = (int64_t)(v & 0xffffffffull);
    idx_t[k] = (int64_t)(v >> 32);
  }
  if (k <= n_cols) {
    int64_t lo = 0, hi = n_edges;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if ((int64_t)sorted_key[mid] < k) lo = mid + 1;
      else hi = mid;
    }
    ptr_t[k] = lo;
  }
}

__global__ void fill_i64_kernel(int64_t* __restrict__ out, int64_t n, int64_t value) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k < n) out[k] = value;
}

// One wave per row: val[e] = 1 / deg(row) for the row's edges.
__global__ void edge_value_degree_kernel(const int64_t* __restrict__ ptr, int64_t n_rows,
                                         float* __restrict__ out) {
  const int lane = lane_id();
  const int64_t r = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (r >= n_rows) return;
  const int64_t b = ptr[r], e = ptr[r + 1];
  if (e <= b) return;
  const float v = 1.0f / (float)(e - b);
  for (int64_t i = b + lane; i < e; i += CXG_WAVE) out[i] = v;
}

__global__ void pad_rel_kernel(int64_t* __restrict__ rel, int64_t* __restrict__ idx,
                               const int64_t* __restrict__ count, int thres, int num_rel,
                               int64_t base) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t slots = (int64_t)num_rel * (thres - 1);
  if (t >= slots) return;
  const int which = (int)(t / (thres - 1));
  const int64_t mod = count[which] % thres;
  const bool fill = (mod != 0) && ((t % (thres - 1)) < (thres - mod));
  rel[base + t] = fill ? which : num_rel;
  if (idx) idx[base + t] = -1;
}

// Transposed graph of an edge prefix from the transposed graph of the whole edge array.
// A stable sort by source keeps every source's edges in position order, so the entries of
// the prefix [0, limit) are, per source, the leading ones: the prefix graph is the stable
// compaction of the entries with perm < limit -- one scan and one scatter instead of a sort.
struct EntryInPrefix {
  const int64_t* perm;
  int64_t n_entries, limit;
  __device__ int64_t operator()(int64_t k) const { return (k < n_entries && perm[k] < limit) ? 1 : 0; }
};

__global__ void transpose_prefix_fill_kernel(const int64_t* __restrict__ ptr_t_all,
                                             const int64_t* __restrict__ idx_t_all,
                                             const int64_t* __restrict__ perm_all, int64_t n_entries,
                                             int64_t limit, int64_t n_cols, const int64_t* __restrict__ pos,
                                             int64_t* __restrict__ ptr_t, int64_t* __restrict__ idx_t,
                                             int64_t* __restrict__ perm) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k < n_entries) {
    const int64_t p = perm_all[k];
    if (p < limit) {
      const int64_t o = pos[k];
      idx_t[o] = idx_t_all[k];
      perm[o] = p;
    }
  }
  if (k <= n_cols) ptr_t[k] = pos[ptr_t_all[k]];
}

// rocPRIM sorts up to 2^20 items by merge sort whatever the key width: one block sort and
// log2(n / 4096) merge passes of two kernels each -- 22 launches of a few microseconds for
// the 936 k edges of a sampled batch, whose keys have 20 significant bits.  Its radix sort
// takes one pass per 8 key bits, so it is used from 2^16 items on (the reversed graph of the
// largest layer of a sampled batch, sort and fills: 0.260 -> 0.225 ms).
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, (size_t)1 << 16>;

int bits_for(int64_t n) {
  int b = 1;
  while (b < 63 && ((int64_t)1 << b) < n) ++b;
  return b;
}

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

constexpr int64_t kNarrowLimit = (int64_t)1 << 32;

size_t narrow_sort_temp_bytes(int64_t n_edges, int64_t n_cols) {
  size_t temp = 0;
  ColumnKeyIter keys(nullptr, ColumnKey());
  hipError_t e = rocprim::radix_sort_pairs<cxg::SortConfig>(nullptr, temp, keys, (uint32_t*)nullptr,
                                           (const uint64_t*)nullptr, (uint64_t*)nullptr,
                                           (size_t)n_edges, 0, bits_for(n_cols > 1 ? n_cols : 2),
                                           (hipStream_t)0);
  return e == hipSuccess ? temp : 0;
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_csr_transpose_workspace_bytes(int64_t n_edges, int64_t n_cols) {
  if (n_edges < 0 || n_cols < 0) return 0;
  size_t temp = 0;
  rocprim::counting_iterator<int64_t> iota(0);
  hipError_t e = rocprim::radix_sort_pairs<cxg::SortConfig>(nullptr, temp, (const int64_t*)nullptr, (int64_t*)nullptr,
                                           iota, (int64_t*)nullptr, (size_t)n_edges, 0,
                                           cxg::bits_for(n_cols > 1 ? n_cols : 2), (hipStream_t)0);
  if (e != hipSuccess) return 0;
  const size_t narrow = cxg::narrow_sort_temp_bytes(n_edges, n_cols);
  if (narrow > temp) temp = narrow;      // the narrow form's keys need half the room of the wide ones
  return cxg::align256((size_t)n_edges * sizeof(int64_t)) + cxg::align256(temp) + 256;
}

int cxg_csr_transpose_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows, int64_t n_cols,
                          int64_t n_edges, int64_t* ptr_t, int64_t* idx_t, int64_t* perm,
                          void* workspace, size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_cols >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr && ptr_t, CXG_ERR_ARG, "null ptr");
  CXG_REQUIRE(n_edges == 0 || (idx && idx_t && perm), CXG_ERR_ARG, "null idx/idx_t/perm");
  const size_t need = cxg_csr_transpose_workspace_bytes(n_edges, n_cols);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  int64_t* sorted_src = reinterpret_cast<int64_t*>(workspace);
  const size_t off = cxg::align256((size_t)n_edges * sizeof(int64_t));
  void* temp = reinterpret_cast<char*>(workspace) + off;
  size_t temp_bytes = workspace_bytes - off;
  if (n_edges == 0) {
    hipLaunchKernelGGL(cxg::fill_i64_kernel, dim3((unsigned)cxg::ceil_div(n_cols + 1, cxg::kBlock)),
                       dim3(cxg::kBlock), 0, st, ptr_t, n_cols + 1, (int64_t)0);
    CXG_LAUNCH_CHECK("fill_i64_kernel");
    return CXG_OK;
  }
  if (n_rows < cxg::kNarrowLimit && n_cols < cxg::kNarrowLimit && n_edges < cxg::kNarrowLimit) {
    const dim3 grid((unsigned)cxg::ceil_div(n_edges, cxg::kBlock)), block(cxg::kBlock);
    uint64_t* packed = reinterpret_cast<uint64_t*>(idx_t);      // outputs double as sort buffers
    uint32_t* sorted_key = reinterpret_cast<uint32_t*>(workspace);
    const dim3 wgrid((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges, cxg::kRowSpan), cxg::kBlock / CXG_WAVE));
    hipLaunchKernelGGL(cxg::expand_rows_kernel<1>, wgrid, block, 0, st, ptr, n_rows, n_edges,
                       (void*)packed);
    CXG_LAUNCH_CHECK("expand_rows_kernel");
    cxg::ColumnKeyIter keys(idx, cxg::ColumnKey());
    CXG_HIP_CHECK(rocprim::radix_sort_pairs<cxg::SortConfig>(temp, temp_bytes, keys, sorted_key, packed,
                                            reinterpret_cast<uint64_t*>(perm), (size_t)n_edges, 0,
                                            cxg::bits_for(n_cols > 1 ? n_cols : 2), st));
    const int64_t work = (n_edges > n_cols + 1) ? n_edges : n_cols + 1;
    hipLaunchKernelGGL(cxg::transpose_unpack_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)), block, 0,
                       st, sorted_key, n_edges, n_cols, perm, idx_t, ptr_t);
    CXG_LAUNCH_CHECK("transpose_unpack_kernel");
    return CXG_OK;
  }
  if (n_edges > 0) {
    rocprim::counting_iterator<int64_t> iota(0);
    CXG_HIP_CHECK(rocprim::radix_sort_pairs<cxg::SortConfig>(temp, temp_bytes, idx, sorted_src, iota, perm,
                                            (size_t)n_edges, 0, cxg::bits_for(n_cols > 1 ? n_cols : 2),
                                            st));
  }
  const int64_t work = (n_edges > n_cols + 1) ? n_edges : n_cols + 1;
  hipLaunchKernelGGL(cxg::transpose_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, st, ptr, n_rows, sorted_src, perm, n_edges, n_cols, ptr_t,
                     idx_t);
  CXG_LAUNCH_CHECK("transpose_fill_kernel");
  return CXG_OK;
}

size_t cxg_csr_transpose_prefix_workspace_bytes(int64_t n_edges_all) {
  if (n_edges_all < 0) return 0;
  size_t temp = 0;
  cxg::EntryInPrefix f{nullptr, 0, 0};
  auto in = rocprim::make_transform_iterator(rocprim::counting_iterator<int64_t>(0), f);
  if (rocprim::exclusive_scan(nullptr, temp, in, (int64_t*)nullptr, (int64_t)0, (size_t)(n_edges_all + 1),
                              rocprim::plus<int64_t>(), (hipStream_t)0) != hipSuccess)
    return 0;
  return cxg::align256((size_t)(n_edges_all + 1) * sizeof(int64_t)) + cxg::align256(temp) + 256;
}

int cxg_csr_transpose_prefix_i64(const int64_t* ptr_t_all, const int64_t* idx_t_all, const int64_t* perm_all,
                                 int64_t n_edges_all, int64_t edge_limit, int64_t n_cols, int64_t* ptr_t,
                                 int64_t* idx_t, int64_t* perm, void* workspace, size_t workspace_bytes,
                                 void* stream) {
  CXG_REQUIRE(n_edges_all >= 0 && edge_limit >= 0 && n_cols >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(edge_limit <= n_edges_all, CXG_ERR_ARG, "edge_limit %lld exceeds the %lld edges of the whole graph",
              (long long)edge_limit, (long long)n_edges_all);
  CXG_REQUIRE(ptr_t_all && ptr_t, CXG_ERR_ARG, "null ptr_t");
  CXG_REQUIRE(n_edges_all == 0 || (idx_t_all && perm_all), CXG_ERR_ARG, "null idx_t_all/perm_all");
  CXG_REQUIRE(edge_limit == 0 || (idx_t && perm), CXG_ERR_ARG, "null idx_t/perm");
  const size_t need = cxg_csr_transpose_prefix_workspace_bytes(n_edges_all);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  int64_t* pos = reinterpret_cast<int64_t*>(workspace);
  const size_t off = cxg::align256((size_t)(n_edges_all + 1) * sizeof(int64_t));
  void* temp = reinterpret_cast<char*>(workspace) + off;
  size_t temp_bytes = workspace_bytes - off;
  cxg::EntryInPrefix f{perm_all, n_edges_all, edge_limit};
  auto in = rocprim::make_transform_iterator(rocprim::counting_iterator<int64_t>(0), f);
  CXG_HIP_CHECK(rocprim::exclusive_scan(temp, temp_bytes, in, pos, (int64_t)0, (size_t)(n_edges_all + 1),
                                        rocprim::plus<int64_t>(), st));
  const int64_t work = (n_edges_all > n_cols + 1) ? n_edges_all : n_cols + 1;
  hipLaunchKernelGGL(cxg::transpose_prefix_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, st, ptr_t_all, idx_t_all, perm_all, n_edges_all, edge_limit, n_cols,
                     pos, ptr_t, idx_t, perm);
  CXG_LAUNCH_CHECK("transpose_prefix_fill_kernel");
  return CXG_OK;
}

int cxg_csr_row_ids_i64(const int64_t* ptr, int64_t n_rows, int64_t n_edges, int64_t* rows,
                        void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  if (n_edges == 0) return CXG_OK;
  CXG_REQUIRE(ptr && rows, CXG_ERR_ARG, "null pointer");
  const dim3 wgrid((unsigned)cxg::ceil_div(cxg::ceil_div(n_edges, cxg::kRowSpan), cxg::kBlock / CXG_WAVE));
  hipLaunchKernelGGL(cxg::expand_rows_kernel<0>, wgrid, dim3(cxg::kBlock), 0,
                     reinterpret_cast<hipStream_t>(stream), ptr, n_rows, n_edges, (void*)rows);
  CXG_LAUNCH_CHECK("expand_rows_kernel");
  return CXG_OK;
}

int cxg_edge_value_degree_f32(const int64_t* ptr, int64_t n_rows, float* out, void* stream) {
  CXG_REQUIRE(n_rows >= 0, CXG_ERR_ARG, "negative size");
  if (n_rows == 0) return CXG_OK;
  CXG_REQUIRE(ptr && out, CXG_ERR_ARG, "null pointer");
  const int64_t threads = n_rows * CXG_WAVE;
  hipLaunchKernelGGL(cxg::edge_value_degree_kernel,
                     dim3((unsigned)cxg::ceil_div(threads, cxg::kBlock)), dim3(cxg::kBlock), 0,
                     reinterpret_cast<hipStream_t>(stream), ptr, n_rows, out);
  CXG_LAUNCH_CHECK("edge_value_degree_kernel");
  return CXG_OK;
}

int cxg_pad_rel_i64(int64_t* rel, int64_t* idx, const int64_t* count, int thres, int num_rel,
                    int64_t base, void* stream) {
  CXG_REQUIRE(thres >= 1 && num_rel >= 0 && base >= 0, CXG_ERR_ARG, "bad thres/num_rel/base");
  const int64_t slots = (int64_t)num_rel * (thres - 1);
  if (slots == 0) return CXG_OK;
  CXG_REQUIRE(rel && count, CXG_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(cxg::pad_rel_kernel, dim3((unsigned)cxg::ceil_div(slots, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), rel, idx, count, thres,
                     num_rel, base);
  CXG_LAUNCH_CHECK("pad_rel_kernel");
  return CXG_OK;
}

}  // extern "C"
