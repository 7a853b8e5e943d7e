// Shared host/device helpers for the gfx950 graph kernels.
//
// Everything here assumes a 64-lane wavefront (CDNA).  Error reporting: every
// extern "C" entry point returns 0 on success or a negative cxg_status code and
// stores a human-readable message retrievable with cxg_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/cxgnn_hip.h"

#define CXG_WAVE 64

namespace cxg {

int set_error(int code, const char* fmt, ...);

#define CXG_REQUIRE(cond, code, ...)                 \
  do {                                               \
    if (!(cond)) return cxg::set_error((code), __VA_ARGS__); \
  } while (0)

#define CXG_HIP_CHECK(expr)                                                   \
  do {                                                                        \
    hipError_t _e = (expr);                                                   \
    if (_e != hipSuccess)                                                     \
      return cxg::set_error(CXG_ERR_HIP, "%s failed: %s (%s:%d)", #expr,      \
                            hipGetErrorString(_e), __FILE__, __LINE__);       \
  } while (0)

#define CXG_LAUNCH_CHECK(name)                                                \
  do {                                                                        \
    hipError_t _e = hipGetLastError();                                        \
    if (_e != hipSuccess)                                                     \
      return cxg::set_error(CXG_ERR_HIP, "launch of %s failed: %s", name,     \
                            hipGetErrorString(_e));                           \
  } while (0)

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

#ifdef __HIPCC__
__device__ __forceinline__ int lane_id() { return threadIdx.x & (CXG_WAVE - 1); }

// Broadcast the value held by `lane` (wave-uniform lane number) to an SGPR.
__device__ __forceinline__ int bcast_i32(int v, int lane) {
  return __builtin_amdgcn_readlane(v, lane);
}
__device__ __forceinline__ float bcast_f32(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ int64_t bcast_i64(int64_t v, int lane) {
  int lo = __builtin_amdgcn_readlane((int)(v & 0xffffffffll), lane);
  int hi = __builtin_amdgcn_readlane((int)(v >> 32), lane);
  return ((int64_t)hi << 32) | (uint32_t)lo;
}
__device__ __forceinline__ int uniform_i32(int v) {
  return __builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ int64_t uniform_i64(int64_t v) {
  int lo = __builtin_amdgcn_readfirstlane((int)(v & 0xffffffffll));
  int hi = __builtin_amdgcn_readfirstlane((int)(v >> 32));
  return ((int64_t)hi << 32) | (uint32_t)lo;
}

// Streaming accesses: data read or written once (index and value streams, output rows) is
// marked non-temporal, so that in the 4 MB L2 of an XCD it does not push out the source rows
// that many edges share.
template <typename T> __device__ __forceinline__ T stream_load(const T* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void stream_store(float* p, float v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void stream_store(float* p, float2 v) {
  typedef float f2_t __attribute__((ext_vector_type(2)));
  f2_t t = {v.x, v.y};
  __builtin_nontemporal_store(t, reinterpret_cast<f2_t*>(p));
}
__device__ __forceinline__ void stream_store(float* p, float4 v) {
  typedef float f4_t __attribute__((ext_vector_type(4)));
  f4_t t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<f4_t*>(p));
}
// First index i in [0, n) with a[i] >= key (n if none); `a` is non-decreasing.
// All 64 lanes cooperate: each round probes 64 evenly spaced elements, so the
// search finishes in ceil(log64(n)) dependent memory round trips.
template <typename T>
__device__ __forceinline__ int64_t wave_lower_bound(const T* __restrict__ a,
                                                    int64_t n, int64_t key) {
  int64_t lo = 0, hi = n;
  const int lane = lane_id();
  while (hi > lo) {
    const int64_t len = hi - lo;
    const int64_t step = (len + CXG_WAVE - 1) / CXG_WAVE;
    const int64_t probe = lo + (int64_t)lane * step;
    bool less = false;
    if (probe < hi) less = (int64_t)a[probe] < key;
    const int cnt = __popcll(__ballot(less));
    if (cnt == 0) {
      hi = lo;
    } else {
      const int64_t last_true = lo + (int64_t)(cnt - 1) * step;
      const int64_t nhi = last_true + step;
      lo = last_true + 1;
      hi = nhi < hi ? nhi : hi;
    }
  }
  return uniform_i64(lo);
}

// Rows of consecutive edge positions, one position per lane, for a wave that walks
// forward through the edge array: row(p) = the r with ptr[r] <= p < ptr[r+1].  The wave
// keeps the ends of 64 rows (relative to its first position) in one register per lane;
// a position is located by a six-step search through lane shuffles, and only when a
// position lies past the window is the window moved, by one cooperative search of ptr.
struct RowWalker {
  const int64_t* ptr;
  int64_t n_rows, p0, rbase;
  int ends;                                  // ptr[rbase + 1 + lane] - p0, clamped

  __device__ __forceinline__ void load_window() {
    const int64_t k = rbase + 1 + lane_id();
    const int64_t d = k <= n_rows ? ptr[k] - p0 : (int64_t)(1 << 30);   // past the last row: never reached
    ends = d > (int64_t)(1 << 30) ? (1 << 30) : (int)d;
  }
  __device__ __forceinline__ void init(const int64_t* ptr_, int64_t n_rows_, int64_t p0_) {
    ptr = ptr_; n_rows = n_rows_; p0 = p0_;
    rbase = wave_lower_bound(ptr, n_rows + 1, p0 + 1) - 1;
    load_window();
  }
  // `rel` = position - p0 (non-decreasing over lanes and over calls, < 2^30);
  // lanes with !valid get -1; positions at or past ptr[n_rows] get n_rows.  Every pass
  // settles at least the first pending lane, so 64 passes always suffice; the bound
  // makes the loop end on a ptr that is not sorted, too.
  __device__ __forceinline__ int64_t row_of(int rel, bool valid) {
    int64_t row = -1;
    for (int pass = 0; pass < CXG_WAVE + 1; ++pass) {
      // the shuffles run with every lane active; only the use of their result is per lane
      const int window_end = __shfl(ends, CXG_WAVE - 1, CXG_WAVE);
      int cnt = 0;                           // window rows whose end is <= rel
#pragma unroll
      for (int step = 32; step >= 1; step >>= 1)
        if (__shfl(ends, cnt + step - 1, CXG_WAVE) <= rel) cnt += step;
      if (row < 0 && valid && window_end > rel) row = rbase + cnt;
      const unsigned long long pending = __ballot(valid && row < 0);
      if (pending == 0) break;
      const int first = __ffsll((long long)pending) - 1;
      const int64_t target = p0 + __shfl(rel, first, CXG_WAVE);
      rbase = wave_lower_bound(ptr, n_rows + 1, target + 1) - 1;
      load_window();
    }
    return row;
  }
};
#endif  // __HIPCC__

}  // namespace cxg
