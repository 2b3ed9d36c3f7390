// Small fp16 helpers shared by the quantizers: packed minimum / maximum on raw words and exact widening
// through the mixed-precision FMA, which cost no conversion instruction (v_cvt_f32_f16 issues at half
// the rate of plain vector instructions on this part).
#pragma once
#include "kitty_common.h"

namespace kitty {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
// Half `hi` (0 / 1) of a word of two fp16 numbers, as the compiler's half type: widened where it is used,
// it enters a mixed-precision FMA as it is (exactly, subnormals included) and costs no conversion.
__device__ __forceinline__ _Float16 half_of(uint32_t w, int hi) {
  const half2_t p = __builtin_bit_cast(half2_t, w);
  return hi ? p.y : p.x;
}
// Packed fp16 minimum / maximum of two words.  Written out because the compiler first re-quiets every
// operand it has not produced itself (one more instruction per loaded word); fp16 numbers order as
// their fp32 values do, and a quiet NaN loses against a number as in fminf / fmaxf.
__device__ __forceinline__ uint32_t pk_min_f16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_min_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ uint32_t pk_max_f16(uint32_t a, uint32_t b) {
  uint32_t d;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}

// |a| + |b| in fp32 and a widened to fp32, for half `hi` of the words a and b: one mixed-precision FMA
// each, which widens its fp16 operands exactly (subnormals included) on the way in.  (x + -0 = x for
// every x, -0 included.)
__device__ __forceinline__ float abs_sum_f16(uint32_t a, uint32_t b, int hi) {
  float d;
  if (hi) asm("v_fma_mix_f32 %0, |%1|, 1.0, |%2| op_sel:[1,0,1] op_sel_hi:[1,0,1]" : "=v"(d) : "v"(a), "v"(b));
  else asm("v_fma_mix_f32 %0, |%1|, 1.0, |%2| op_sel:[0,0,0] op_sel_hi:[1,0,1]" : "=v"(d) : "v"(a), "v"(b));
  return d;
}
__device__ __forceinline__ float widen_f16(uint32_t a, int hi) {
  float d;
  const float neg_zero = -0.0f;
  if (hi) asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(a), "s"(neg_zero));
  else asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(a), "s"(neg_zero));
  return d;
}

// Half `hi` of the word a, widened exactly, times the fp32 number r: the product rounded once to fp32,
// as v_mul_f32 of the widened value gives it (the -0 addend keeps a zero product's sign).
__device__ __forceinline__ float mul_f16_f32(uint32_t a, int hi, float r) {
  float d;
  const float neg_zero = -0.0f;
  if (hi) asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(a), "v"(r), "s"(neg_zero));
  else asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(d) : "v"(a), "v"(r), "s"(neg_zero));
  return d;
}

}  // namespace kitty
