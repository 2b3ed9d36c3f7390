// Arithmetic shared by the quantize-and-pack kernels (the page-sized ones and those for other head
// dimensions): the boost score's single fp16 rounding and the group quantizer's IEEE fp32 division.
// Contract: kitty_quant_pack.py:75-82, 106-112, 201-204, 227-230, 280.
#pragma once
#include "kitty_common.h"

namespace kitty {

// fp16 bit pattern of (S * 2^-31) rounded to nearest even, S = sum over 128 tokens of |x| * 2^24,
// i.e. the mean of |x| rounded once.  Positive fp16 patterns order like their values.
__device__ inline uint16_t mean_abs_fp16_bits(uint64_t S) {
  if (S == 0) return 0;
  int msb = 63 - __clzll((long long)S);
  int E = msb - 31;
  if (E >= -14) {
    int shift = msb - 10;
    uint64_t q;
    if (shift > 0) {
      q = S >> shift;
      uint64_t rem = S & ((1ull << shift) - 1), half = 1ull << (shift - 1);
      if (rem > half || (rem == half && (q & 1))) q++;
    } else {
      q = S << (-shift);
    }
    if (q == 2048) { q = 1024; E++; }
    if (E > 15) return 0x7C00;
    return (uint16_t)(((uint32_t)(E + 15) << 10) | (uint32_t)(q & 1023));
  }
  uint64_t q = S >> 7, rem = S & 127;
  if (rem > 64 || (rem == 64 && (q & 1))) q++;
  return (uint16_t)q;
}

__device__ inline float h2f(uint16_t bits) { return __half2float(__ushort_as_half(bits)); }

// IEEE fp32 division by a divisor that is shared by a whole group.  This is the correctly rounded
// sequence the compiler emits for `/` (reciprocal, one Newton step, quotient, two residual
// corrections) without its range scaling and special-case fix-up, which cannot trigger here: the
// divisor is a scale in [1e-6, 4.4e4], the dividend x - min is 0 or in [2^-24, 1.4e5].  The
// reciprocal part depends on the divisor only and is computed once per group.  Bit-identical to
// `/` on that domain except that -0 / d gives +0, which the + 0.5 that follows erases.
struct Divisor {
  float d, r;
};
__device__ __forceinline__ Divisor make_divisor(float d) {
  float r = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, r, 1.0f);
  r = __builtin_fmaf(e, r, r);
  return {d, r};
}
__device__ __forceinline__ float div_by(float n, Divisor k) {
  float q = n * k.r;
  float rem = __builtin_fmaf(-k.d, q, n);
  q = __builtin_fmaf(rem, k.r, q);
  rem = __builtin_fmaf(-k.d, q, n);
  return __builtin_fmaf(rem, k.r, q);
}
// floor(min(x / scale + 0.5, qmax + 0.5)) as a float: the code.  x >= 0, so the lower clamp of
// the reference never acts, and clamping before the floor gives the same integer.
__device__ __forceinline__ float code_of(float x_minus_min, Divisor k, float qlim) {
  return __builtin_floorf(fminf(div_by(x_minus_min, k) + 0.5f, qlim));
}
}  // namespace kitty
