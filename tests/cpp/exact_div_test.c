// Host check of the division the fp8 quantizers use (ksanallm_amd/csrc/fp8_quant.hip, ExactDiv):
//     y = 1 / s (correctly rounded),  q0 = x * y,  r = fma(-q0, s, x),  q = copysign(fma(r, y, q0), x)
// must equal x / s bit for bit wherever the e4m3 conversion can tell the difference: for 2^-80 <= s <= 2^100 (the range
// the kernels take this path for) and |x / s| >= 2^-20, and for x = +-0.  Below that r may leave the normal range and q
// be one unit in the last place off, which still converts to the same signed zero (e4m3's smallest step is 2^-9).
// Scaling x or s by a power of two changes nothing in any of these operations while all intermediates stay normal, so
// mantissas are what matters: every one of the 2^23 mantissas of s against every x with up to 11 fraction bits (fp16
// has 10, bf16 7), then a band of exponents and signs on a sample of scales, and the scales the group quantizer
// actually forms (amax / 448 for every positive bf16 amax from 2^-30 to 2^30).
// Exit status 0 = no mismatch.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

static inline float from_bits(uint32_t b) {
  float f;
  memcpy(&f, &b, 4);
  return f;
}
static inline int same(float a, float b) { return memcmp(&a, &b, 4) == 0; }
static inline float fast_div(float x, float s, float y) {
  const float q0 = x * y;
  const float r = fmaf(-q0, s, x);
  return copysignf(fmaf(r, y, q0), x);
}

int main(void) {
  long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(dynamic, 4096)
  for (uint32_t sm = 0; sm < (1u << 23); ++sm) {
    const float s = from_bits((127u << 23) | sm);
    const float y = 1.0f / s;
    for (uint32_t xm = 0; xm < (1u << 11); ++xm) {
      const float x = from_bits((127u << 23) | (xm << 12));
      if (!same(x / s, fast_div(x, s, y))) ++bad;
    }
  }
  printf("all scale mantissas x all 11-bit inputs: %ld mismatches\n", bad);

  // exponents and signs: scales from 2^-80 to 2^100, quotients from 2^-20 up to the clamp exactly, smaller ones
  // to within the zero of e4m3, -0
  long bad2 = 0;
#pragma omp parallel for reduction(+ : bad2) schedule(dynamic, 64)
  for (uint32_t i = 0; i < (1u << 15); ++i) {
    const uint32_t sm = (i * 257u + 11u) & 0x7fffffu;
    for (int se = -80; se <= 100; se += 15) {
      const float s = from_bits(((uint32_t)(127 + se) << 23) | sm);
      const float y = 1.0f / s;
      for (int xe = se - 20; xe <= se + 9; xe += 1) {
        if (xe > 120) continue;
        for (uint32_t xm = 0; xm < (1u << 11); xm += 3) {
          const float x = from_bits(((uint32_t)(127 + xe) << 23) | (xm << 12));
          if (!same(x / s, fast_div(x, s, y)) || !same(-x / s, fast_div(-x, s, y))) ++bad2;
        }
      }
      for (int xe = se - 60; xe < se - 20; xe += 3) {
        if (xe < -126) continue;
        for (uint32_t xm = 0; xm < (1u << 11); xm += 31) {
          const float x = from_bits(((uint32_t)(127 + xe) << 23) | (xm << 12));
          const float f = fast_div(-x, s, y);
          if (!(f <= 0.0f && f > -0x1p-18f && signbit(f))) ++bad2;  // converts to -0 like the true quotient
        }
      }
      if (!same(-0.0f / s, fast_div(-0.0f, s, y)) || !same(0.0f / s, fast_div(0.0f, s, y))) ++bad2;
    }
  }
  printf("exponent and sign band: %ld mismatches\n", bad2);

  // the scales of the group quantizer: amax / 448 for every positive bf16 amax in [2^-30, 2^30], inputs below amax
  long bad3 = 0;
#pragma omp parallel for reduction(+ : bad3) schedule(dynamic, 16)
  for (uint32_t ab = 0x3080u; ab <= 0x4e80u; ++ab) {  // bf16 bit patterns
    const float amax = from_bits(ab << 16);
    const float s = amax / 448.0f;
    const float y = 1.0f / s;
    for (uint32_t xb = ab > 0x0c00u ? ab - 0x0c00u : 1; xb <= ab; ++xb) {
      const float x = from_bits(xb << 16);
      if (!same(x / s, fast_div(x, s, y))) ++bad3;
    }
  }
  printf("group-quantizer scales (bf16): %ld mismatches\n", bad3);
  return (bad | bad2 | bad3) != 0;
}
