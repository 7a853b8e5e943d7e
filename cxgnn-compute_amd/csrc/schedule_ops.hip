// Scheduling helpers as device index work: degree bucketing (neighbor grouping),
// row / edge filtering of a CSR graph (also the per-relation sub-graphs of
// rel_schedule) and COO -> CSR.  The reference runs these as Python or C++ loops
// over rows on the host (cxgnncomp/schedule.py:6-35,106-144,
// src/cpp/src/schedule.cu:5-63); here every step is an exclusive scan (rocPRIM)
// followed by a fill kernel with one thread per output element.  Results are
// bit-exact functions of the inputs.
//
// Output sizes depend on the data, so each operation is split in two calls: a
// "plan" that leaves the scanned offsets on the device (their last entry is the
// output size, which the caller reads back to allocate), and a "fill".
#include "cxg_common.hpp"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/iterator/counting_iterator.hpp>
#include <rocprim/iterator/transform_iterator.hpp>

namespace cxg {
namespace {

// rocPRIM sorts up to 2^20 items by merge sort whatever the key width (a block sort and
// log2(n / 4096) merge passes of two kernels each); its radix sort takes one pass per 8
// significant key bits, so it is used from 2^16 items on.
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, (size_t)1 << 16>;


constexpr int kBlock = 256;

size_t align256(size_t x) { return (x + 255) / 256 * 256; }

int bits_for(int64_t n) {
  int b = 1;
  while (b < 63 && ((int64_t)1 << b) < n) ++b;
  return b;
}

// Largest r in [0, n) with off[r] <= k, for a non-decreasing off[0..n].
__device__ __forceinline__ int64_t owner_of(const int64_t* __restrict__ off, int64_t n, int64_t k) {
  int64_t lo = 0, hi = n + 1;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (off[mid] <= k) lo = mid + 1;
    else hi = mid;
  }
  return lo - 1;
}

// ---- functors scanned by the plan calls (element i of an n+1 long sequence) ----
struct GroupsOfRow {
  const int64_t* ptr;
  int64_t n_rows;
  int64_t thres;
  __device__ int64_t operator()(int64_t i) const {
    if (i >= n_rows) return 0;
    const int64_t g = (ptr[i + 1] - ptr[i] + thres - 1) / thres;
    return g > 0 ? g : 1;                     // an empty row is one empty group
  }
};
struct KeptRow {
  const uint8_t* remove;
  int64_t n_rows;
  __device__ int64_t operator()(int64_t i) const { return (i < n_rows && !remove[i]) ? 1 : 0; }
};
struct KeptRowEdges {
  const int64_t* ptr;
  const uint8_t* remove;
  int64_t n_rows;
  __device__ int64_t operator()(int64_t i) const {
    return (i < n_rows && !remove[i]) ? ptr[i + 1] - ptr[i] : 0;
  }
};
struct KeptEdge {
  const uint8_t* remove;
  const int32_t* rel;
  int32_t keep_rel;
  int64_t n_edges;
  __device__ int64_t operator()(int64_t e) const {
    if (e >= n_edges) return 0;
    return rel ? (rel[e] == keep_rel ? 1 : 0) : (remove[e] ? 0 : 1);
  }
};
struct RowWithKeptEdges {
  const int64_t* ptr;
  const int64_t* edge_pos;
  int64_t n_rows;
  __device__ int64_t operator()(int64_t i) const {
    return (i < n_rows && edge_pos[ptr[i + 1]] > edge_pos[ptr[i]]) ? 1 : 0;
  }
};

template <class F>
hipError_t scan_of(void* temp, size_t& temp_bytes, F f, int64_t* out, int64_t count, hipStream_t st) {
  auto in = rocprim::make_transform_iterator(rocprim::counting_iterator<int64_t>(0), f);
  return rocprim::exclusive_scan(temp, temp_bytes, in, out, (int64_t)0, (size_t)count,
                                 rocprim::plus<int64_t>(), st);
}

__global__ void neighbor_group_fill_kernel(const int64_t* __restrict__ ptr,
                                           const int64_t* __restrict__ group_off, int64_t n_rows,
                                           int64_t thres, int64_t n_groups,
                                           int64_t* __restrict__ new_ptr,
                                           int64_t* __restrict__ new_target) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g == 0) new_ptr[0] = 0;
  if (g >= n_groups) return;
  const int64_t r = owner_of(group_off, n_rows, g);
  const int64_t k = g - group_off[r];
  const int64_t end = ptr[r] + (k + 1) * thres;
  new_target[g] = r;
  new_ptr[g + 1] = end < ptr[r + 1] ? end : ptr[r + 1];
}

__global__ void filter_rows_fill_kernel(const int64_t* __restrict__ ptr, const int64_t* __restrict__ idx,
                                        int64_t n_rows, const int64_t* __restrict__ row_off,
                                        const int64_t* __restrict__ edge_off, int64_t n_edges_out,
                                        int64_t* __restrict__ new_ptr, int64_t* __restrict__ new_idx) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k == 0) new_ptr[0] = 0;
  if (k < n_rows && row_off[k + 1] > row_off[k]) new_ptr[row_off[k] + 1] = edge_off[k + 1];
  if (k < n_edges_out) {
    const int64_t r = owner_of(edge_off, n_rows, k);
    new_idx[k] = idx[ptr[r] + (k - edge_off[r])];
  }
}

__global__ void filter_edges_fill_kernel(const int64_t* __restrict__ ptr, const int64_t* __restrict__ idx,
                                         int64_t n_rows, int64_t n_edges,
                                         const int64_t* __restrict__ edge_pos,
                                         const int64_t* __restrict__ row_off,
                                         int64_t* __restrict__ new_ptr, int64_t* __restrict__ new_idx,
                                         int64_t* __restrict__ new_target) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k == 0) new_ptr[0] = 0;
  if (k < n_rows && row_off[k + 1] > row_off[k]) {
    new_ptr[row_off[k] + 1] = edge_pos[ptr[k + 1]];
    if (new_target) new_target[row_off[k]] = k;
  }
  if (k < n_edges && edge_pos[k + 1] > edge_pos[k]) new_idx[edge_pos[k]] = idx[k];
}

__global__ void coo_fill_kernel(const int64_t* __restrict__ src, const int64_t* __restrict__ sorted_dst,
                                const int64_t* __restrict__ perm, int64_t n_edges, int64_t n_rows,
                                int64_t* __restrict__ ptr, int64_t* __restrict__ idx) {
  const int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (k < n_edges) idx[k] = src[perm[k]];
  if (k <= n_rows) {
    int64_t lo = 0, hi = n_edges;          // number of edges with destination < k
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (sorted_dst[mid] < k) lo = mid + 1;
      else hi = mid;
    }
    ptr[k] = lo;
  }
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_scan_workspace_bytes(int64_t n) {
  if (n < 0) return 0;
  size_t temp = 0;
  cxg::KeptRow f{nullptr, 0};
  if (cxg::scan_of(nullptr, temp, f, (int64_t*)nullptr, n + 1, (hipStream_t)0) != hipSuccess) return 0;
  return cxg::align256(temp) + 256;
}

#define CXG_SCAN_PROLOGUE(COUNT)                                                                   \
  const size_t need = cxg_scan_workspace_bytes(COUNT);                                             \
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,                             \
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);                  \
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);                                          \
  size_t temp_bytes = workspace_bytes

int cxg_neighbor_group_plan_i64(const int64_t* ptr, int64_t n_rows, int64_t thres, int64_t* group_off,
                                void* workspace, size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && thres >= 1, CXG_ERR_ARG, "bad n_rows/thres");
  CXG_REQUIRE(ptr && group_off, CXG_ERR_ARG, "null pointer");
  CXG_SCAN_PROLOGUE(n_rows);
  cxg::GroupsOfRow f{ptr, n_rows, thres};
  CXG_HIP_CHECK(cxg::scan_of(workspace, temp_bytes, f, group_off, n_rows + 1, st));
  return CXG_OK;
}

int cxg_neighbor_group_fill_i64(const int64_t* ptr, const int64_t* group_off, int64_t n_rows,
                                int64_t thres, int64_t n_groups, int64_t* new_ptr, int64_t* new_target,
                                void* stream) {
  CXG_REQUIRE(n_rows >= 0 && thres >= 1 && n_groups >= 0, CXG_ERR_ARG, "bad sizes");
  CXG_REQUIRE(ptr && group_off && new_ptr && (n_groups == 0 || new_target), CXG_ERR_ARG, "null pointer");
  const int64_t work = n_groups > 1 ? n_groups : 1;
  hipLaunchKernelGGL(cxg::neighbor_group_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), ptr, group_off, n_rows,
                     thres, n_groups, new_ptr, new_target);
  CXG_LAUNCH_CHECK("neighbor_group_fill_kernel");
  return CXG_OK;
}

int cxg_filter_rows_plan_i64(const int64_t* ptr, int64_t n_rows, const uint8_t* remove_flag,
                             int64_t* row_off, int64_t* edge_off, void* workspace,
                             size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr && row_off && edge_off && (n_rows == 0 || remove_flag), CXG_ERR_ARG, "null pointer");
  CXG_SCAN_PROLOGUE(n_rows);
  cxg::KeptRow fr{remove_flag, n_rows};
  CXG_HIP_CHECK(cxg::scan_of(workspace, temp_bytes, fr, row_off, n_rows + 1, st));
  temp_bytes = workspace_bytes;
  cxg::KeptRowEdges fe{ptr, remove_flag, n_rows};
  CXG_HIP_CHECK(cxg::scan_of(workspace, temp_bytes, fe, edge_off, n_rows + 1, st));
  return CXG_OK;
}

int cxg_filter_rows_fill_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows,
                             const int64_t* row_off, const int64_t* edge_off, int64_t n_edges_out,
                             int64_t* new_ptr, int64_t* new_idx, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges_out >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr && row_off && edge_off && new_ptr, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(n_edges_out == 0 || (idx && new_idx), CXG_ERR_ARG, "null idx/new_idx");
  int64_t work = n_rows > n_edges_out ? n_rows : n_edges_out;
  if (work < 1) work = 1;
  hipLaunchKernelGGL(cxg::filter_rows_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), ptr, idx, n_rows, row_off,
                     edge_off, n_edges_out, new_ptr, new_idx);
  CXG_LAUNCH_CHECK("filter_rows_fill_kernel");
  return CXG_OK;
}

int cxg_filter_edges_plan_i64(const int64_t* ptr, int64_t n_rows, int64_t n_edges,
                              const uint8_t* remove_flag, const int32_t* rel, int32_t keep_rel,
                              int64_t* edge_pos, int64_t* row_off, void* workspace,
                              size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr && edge_pos && row_off, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(n_edges == 0 || remove_flag || rel, CXG_ERR_ARG, "neither remove_flag nor rel given");
  CXG_SCAN_PROLOGUE(n_rows > n_edges ? n_rows : n_edges);
  cxg::KeptEdge fe{remove_flag, rel, keep_rel, n_edges};
  CXG_HIP_CHECK(cxg::scan_of(workspace, temp_bytes, fe, edge_pos, n_edges + 1, st));
  temp_bytes = workspace_bytes;
  cxg::RowWithKeptEdges fr{ptr, edge_pos, n_rows};
  CXG_HIP_CHECK(cxg::scan_of(workspace, temp_bytes, fr, row_off, n_rows + 1, st));
  return CXG_OK;
}

int cxg_filter_edges_fill_i64(const int64_t* ptr, const int64_t* idx, int64_t n_rows, int64_t n_edges,
                              const int64_t* edge_pos, const int64_t* row_off, int64_t* new_ptr,
                              int64_t* new_idx, int64_t* new_target, void* stream) {
  CXG_REQUIRE(n_rows >= 0 && n_edges >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr && edge_pos && row_off && new_ptr, CXG_ERR_ARG, "null pointer");
  CXG_REQUIRE(n_edges == 0 || idx, CXG_ERR_ARG, "null idx");
  int64_t work = n_rows > n_edges ? n_rows : n_edges;
  if (work < 1) work = 1;
  hipLaunchKernelGGL(cxg::filter_edges_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, reinterpret_cast<hipStream_t>(stream), ptr, idx, n_rows, n_edges,
                     edge_pos, row_off, new_ptr, new_idx, new_target);
  CXG_LAUNCH_CHECK("filter_edges_fill_kernel");
  return CXG_OK;
}

size_t cxg_coo_to_csr_workspace_bytes(int64_t n_edges, int64_t n_rows) {
  if (n_edges < 0 || n_rows < 0) return 0;
  size_t temp = 0;
  rocprim::counting_iterator<int64_t> iota(0);
  hipError_t e = rocprim::radix_sort_pairs<cxg::SortConfig>(nullptr, temp, (const int64_t*)nullptr, (int64_t*)nullptr,
                                           iota, (int64_t*)nullptr, (size_t)n_edges, 0,
                                           cxg::bits_for(n_rows > 1 ? n_rows : 2), (hipStream_t)0);
  if (e != hipSuccess) return 0;
  return cxg::align256((size_t)n_edges * sizeof(int64_t)) + cxg::align256(temp) + 256;
}

int cxg_coo_to_csr_i64(const int64_t* src, const int64_t* dst, int64_t n_edges, int64_t n_rows,
                       int64_t* ptr, int64_t* idx, int64_t* perm, void* workspace,
                       size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n_edges >= 0 && n_rows >= 0, CXG_ERR_ARG, "negative size");
  CXG_REQUIRE(ptr, CXG_ERR_ARG, "null ptr");
  CXG_REQUIRE(n_edges == 0 || (src && dst && idx && perm), CXG_ERR_ARG, "null src/dst/idx/perm");
  const size_t need = cxg_coo_to_csr_workspace_bytes(n_edges, n_rows);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  int64_t* sorted_dst = reinterpret_cast<int64_t*>(workspace);
  const size_t off = cxg::align256((size_t)n_edges * sizeof(int64_t));
  void* temp = reinterpret_cast<char*>(workspace) + off;
  size_t temp_bytes = workspace_bytes - off;
  if (n_edges > 0) {
    rocprim::counting_iterator<int64_t> iota(0);
    CXG_HIP_CHECK(rocprim::radix_sort_pairs<cxg::SortConfig>(temp, temp_bytes, dst, sorted_dst, iota, perm, (size_t)n_edges,
                                            0, cxg::bits_for(n_rows > 1 ? n_rows : 2), st));
  }
  const int64_t work = (n_edges > n_rows + 1) ? n_edges : n_rows + 1;
  hipLaunchKernelGGL(cxg::coo_fill_kernel, dim3((unsigned)cxg::ceil_div(work, cxg::kBlock)),
                     dim3(cxg::kBlock), 0, st, src, sorted_dst, perm, n_edges, n_rows, ptr, idx);
  CXG_LAUNCH_CHECK("coo_fill_kernel");
  return CXG_OK;
}

}  // extern "C"
