/* Host check of the short division the KV-cache write kernels use (pa_kv_cache.hip: quantize8,
 * bf16_amax_to_scale): with r one Newton step from ANY first reciprocal within 1 ulp of 1/s,
 *     q0 = x * r;  q = fma(fma(-s, q0, x), r, q0)
 * must be the correctly rounded float quotient x / s (what the compiler's division gives on the host).
 *   1. per-token scales, exhaustively: s = amax / 448 for every bf16 significand of amax, x every bf16 value with
 *      |x| <= amax down to 2^-40 amax;
 *   2. arbitrary scales (a caller's per-tensor scale): random and structured significands, every bf16 significand
 *      of x over 49 exponents; scales whose significand is all ones are excluded (the kernel divides in full there);
 *   3. amax / 448 from the constant reciprocal, for every positive finite bf16 amax (subnormal ones included).
 * Prints the three mismatch counts; exit status 0 when all are zero.  Build with -ffp-contract=off. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static uint64_t rng = 0x9E3779B97F4A7C15ull;
static uint64_t next(void) { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return rng; }

static float short_quotient(float x, float s, float r) {
  const float q0 = x * r;
  return fmaf(fmaf(-s, q0, x), r, q0);
}

int main(int argc, char** argv) {
  const long n_scales = argc > 1 ? atol(argv[1]) : 20000;
  long bad1 = 0, n1 = 0, bad2 = 0, n2 = 0, bad3 = 0;
  for (int ae = -30; ae <= 30; ae += 6)
    for (uint32_t am = 0; am < 128; am++) {
      const float amax = ldexpf(u2f(0x3f800000u | (am << 16)), ae), s = amax / 448.0f, yc = 1.0f / s;
      for (int k = -1; k <= 1; k++) {
        const float y0 = u2f(f2u(yc) + k), r = fmaf(fmaf(-s, y0, 1.0f), y0, y0);
        for (int e = 0; e >= -40; e--)
          for (uint32_t m = 0; m < 128; m++) {
            const float x = ldexpf(u2f(0x3f800000u | (m << 16)), ae + e);
            if (x > amax) continue;
            n1++;
            bad1 += f2u(short_quotient(x, s, r)) != f2u(x / s);
            bad1 += f2u(short_quotient(-x, s, r)) != f2u(-x / s);
          }
      }
    }
  for (long i = 0; i < n_scales; i++) {
    uint32_t sm = (uint32_t)(next() & 0x7fffff);
    switch (i & 7) {
      case 1: sm |= 0x7ff000; break;
      case 2: sm &= 0xfff; break;
      case 3: sm &= 0x7f0000; break;
      case 4: sm |= 0x7fff80; break;
    }
    if (sm == 0x7fffff) continue;
    const float s = u2f(((127 - 40 + (uint32_t)(next() % 80)) << 23) | sm), yc = 1.0f / s;
    for (int k = -1; k <= 1; k++) {
      const float y0 = u2f(f2u(yc) + k), r = fmaf(fmaf(-s, y0, 1.0f), y0, y0);
      for (int e = -24; e <= 24; e++)
        for (uint32_t m = 0; m < 128; m++) {
          float x = ldexpf(u2f(0x3f800000u | (m << 16)), e) * s * 0.37f;
          x = u2f(f2u(x) & 0xffff0000u); /* a bf16 value */
          n2++;
          bad2 += f2u(short_quotient(x, s, r)) != f2u(x / s);
        }
    }
  }
  for (uint32_t b = 1; b < 0x7f80; b++) {
    const float amax = u2f(b << 16);
    bad3 += f2u(short_quotient(amax, 448.0f, 1.0f / 448.0f)) != f2u(amax / 448.0f);
  }
  printf("per-token %ld cases %ld mismatches; arbitrary scales %ld cases %ld mismatches; amax/448 %ld mismatches\n", n1, bad1,
         n2, bad2, bad3);
  return (bad1 || bad2 || bad3) ? 1 : 0;
}
