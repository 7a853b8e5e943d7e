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
#endif  // __HIPCC__

}  // namespace cxg
