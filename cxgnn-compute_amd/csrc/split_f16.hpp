// Two fp32 values times a power-of-two scale as two packed fp16 parts each:
//   hi = fp16(x * scale), lo = fp16(x * scale - hi)      (x * scale is exact, so hi + lo carries 22 bits)
// in four instructions per pair.  v_fma_mixlo_f16 / v_fma_mixhi_f16 form a * b + c in fp32, round once
// and write one half of the destination, and they read a 16-bit operand out of either half of a
// packed register -- so the high parts need no separate multiply and conversion, and the low parts no
// unpacking.  (From `(_Float16)(x * scale)` and `(_Float16)(x * scale - (float)h)` the compiler makes
// seven instructions per pair: it forms every high part twice.)
#pragma once
#include <hip/hip_runtime.h>

namespace cxg {

__device__ __forceinline__ void split_f16_pair(float x0, float x1, float scale, unsigned& hi, unsigned& lo) {
  asm("v_fma_mixlo_f16 %0, %1, %2, 0\n\tv_fma_mixhi_f16 %0, %3, %2, 0" : "=&v"(hi) : "v"(x0), "v"(scale), "v"(x1));
  asm("v_fma_mixlo_f16 %0, %1, %2, -%4 op_sel_hi:[0,0,1]\n\t"
      "v_fma_mixhi_f16 %0, %3, %2, -%4 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
      : "=&v"(lo)
      : "v"(x0), "v"(scale), "v"(x1), "v"(hi));
}

// Bit pattern of the largest magnitude of four values: float maxima with the absolute-value operand
// modifier (a NaN loses against a number; four NaNs read as exponent 255, like an infinity).
__device__ __forceinline__ unsigned abs_max4_bits(float a, float b, float c, float d) {
  const float m = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(a), __builtin_fabsf(b)),
                                  __builtin_fmaxf(__builtin_fabsf(c), __builtin_fabsf(d)));
  return __float_as_uint(m) & 0x7fffffffu;
}

}  // namespace cxg
