// x / s in fp32, correctly rounded, for many x and one s, without a division per element.
//
// One correctly rounded reciprocal y = 1 / s and a residual correction per element,
//     q0 = x * y,   r = fma(-q0, s, x)  (exact),   q = fma(r, y, q0),
// give the correctly rounded quotient (Markstein's theorem) as long as r stays in the normal range;
// tests/cpp/exact_div_test.c checks it against the division for every one of the 2^23 mantissas of s and every
// mantissa a 16-bit input can have.  The sign of x is put back afterwards (x = -0 would otherwise come out as +0).
// Scales outside [2^-80, 2^100] take the division itself; inside, r is exact whenever |x / s| >= 2^-20, and a smaller
// quotient that is one unit in the last place off still converts to the same signed zero in e4m3.
#pragma once

#include <hip/hip_runtime.h>

namespace ksq {

struct ExactDiv {
  float s, y;
  bool fast;
  __device__ __forceinline__ explicit ExactDiv(float scale)
      : s(scale), y(1.0f / scale), fast(scale >= 0x1p-80f && scale <= 0x1p100f) {}
  // |x| finite or NaN; an infinite x needs the caller's attention (r would be NaN)
  __device__ __forceinline__ float operator()(float x) const {
    if (!fast) return x / s;
    const float q0 = x * y;
    const float r = __builtin_fmaf(-q0, s, x);
    return __builtin_copysignf(__builtin_fmaf(r, y, q0), x);
  }
};

}  // namespace ksq
