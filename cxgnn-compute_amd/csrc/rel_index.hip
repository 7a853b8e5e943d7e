// Relation segmentation (bit-exact index work): stable grouping of rows by
// relation id, the preprocessing in front of the typed GEMM.
//
//   perm[k]    = original row of the k-th row in relation order (rows of one
//                relation keep their original order: stable sort),
//   seg_ptr[r] = number of rows whose relation id is < r, r in [0, R].
//
// The reference sorts the (padded) relation ids with torch.sort and counts them
// with torch.bincount (cxgnncomp/typed_linear.py:74-87,143-160,262-283); the
// order inside a relation is unspecified there, here it is the original order.
#include "cxg_common.hpp"

#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

namespace cxg {
namespace {

constexpr int kBlock = 256;

template <typename T>
__global__ void seg_ptr_kernel(const T* __restrict__ sorted, int64_t n, int R,
                               int64_t* __restrict__ seg_ptr) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r > R) return;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)sorted[mid] < r) lo = mid + 1;
    else hi = mid;
  }
  seg_ptr[r] = lo;
}

// rocPRIM sorts up to 2^20 items by merge sort whatever the key width (a block sort and
// log2(n / 4096) merge passes of two kernels each); its radix sort takes one pass per 8
// significant key bits, so it is used from 2^16 items on.
using SortConfig = rocprim::radix_sort_config<rocprim::default_config, rocprim::default_config,
                                              rocprim::default_config, (size_t)1 << 16>;

int bits_for(int64_t n) {
  int b = 1;
  while (b < 62 && ((int64_t)1 << b) < n) ++b;
  return b;
}
size_t align256(size_t x) { return (x + 255) / 256 * 256; }

template <typename T>
size_t ws_bytes(int64_t n, int R) {
  size_t temp = 0;
  rocprim::counting_iterator<int64_t> iota(0);
  hipError_t e = rocprim::radix_sort_pairs<cxg::SortConfig>(nullptr, temp, (const T*)nullptr, (T*)nullptr, iota,
                                           (int64_t*)nullptr, (size_t)n, 0, bits_for(R + 1),
                                           (hipStream_t)0);
  if (e != hipSuccess) return 0;
  return align256((size_t)n * sizeof(T)) + align256(temp) + 256;
}

template <typename T>
int rel_segment(const T* types, int64_t n, int R, int64_t* perm, int64_t* seg_ptr, void* workspace,
                size_t workspace_bytes, void* stream) {
  CXG_REQUIRE(n >= 0 && R >= 1, CXG_ERR_ARG, "bad n/R");
  CXG_REQUIRE(seg_ptr, CXG_ERR_ARG, "null seg_ptr");
  CXG_REQUIRE(n == 0 || (types && perm), CXG_ERR_ARG, "null types/perm");
  const size_t need = ws_bytes<T>(n, R);
  CXG_REQUIRE(workspace && workspace_bytes >= need, CXG_ERR_WORKSPACE,
              "workspace of %zu bytes needed, %zu given", need, workspace_bytes);
  CXG_REQUIRE(((uintptr_t)workspace & 255) == 0, CXG_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  T* sorted = reinterpret_cast<T*>(workspace);
  const size_t off = align256((size_t)n * sizeof(T));
  void* temp = reinterpret_cast<char*>(workspace) + off;
  size_t temp_bytes = workspace_bytes - off;
  if (n > 0) {
    rocprim::counting_iterator<int64_t> iota(0);
    CXG_HIP_CHECK(rocprim::radix_sort_pairs<cxg::SortConfig>(temp, temp_bytes, types, sorted, iota, perm, (size_t)n, 0,
                                            bits_for(R + 1), st));
  }
  hipLaunchKernelGGL(seg_ptr_kernel<T>, dim3((unsigned)ceil_div(R + 1, kBlock)), dim3(kBlock), 0, st,
                     sorted, n, R, seg_ptr);
  CXG_LAUNCH_CHECK("seg_ptr_kernel");
  return CXG_OK;
}

}  // namespace
}  // namespace cxg

extern "C" {

size_t cxg_rel_segment_workspace_bytes(int64_t n, int num_rel, int index_bytes) {
  if (n < 0 || num_rel < 1) return 0;
  return index_bytes == 4 ? cxg::ws_bytes<int32_t>(n, num_rel) : cxg::ws_bytes<int64_t>(n, num_rel);
}

int cxg_rel_segment_i64(const int64_t* types, int64_t n, int num_rel, int64_t* perm, int64_t* seg_ptr,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return cxg::rel_segment<int64_t>(types, n, num_rel, perm, seg_ptr, workspace, workspace_bytes, stream);
}

int cxg_rel_segment_i32(const int32_t* types, int64_t n, int num_rel, int64_t* perm, int64_t* seg_ptr,
                        void* workspace, size_t workspace_bytes, void* stream) {
  return cxg::rel_segment<int32_t>(types, n, num_rel, perm, seg_ptr, workspace, workspace_bytes, stream);
}

}  // extern "C"
