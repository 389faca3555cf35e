/* CPU check of the arithmetic the one-launch quantized linear uses for x / scale: with
 * y = 1.0f / s, q0 = x y, r = fma(-q0, s, x), q = fma(r, y, q0), a NaN result replaced by the
 * true quotient.  For every sampled x (a stride through all 2^32 bit patterns, plus every
 * pattern near rounding ties of the quantized result) and a set of divisors the quotient must
 * carry the same bits as x / s wherever 1/8 <= |x / s| <= 1024, and the same int8 after
 * rounding (half to even and half away from zero) and clamping to [-128, 127] everywhere.
 * Usage: div_by_constant_check <stride>   (stride 1 = all 2^32 values of x per divisor). */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static int q8(float t, int even) {
  const float r = even ? rintf(t) : roundf(t);
  return (int)fminf(fmaxf(r, -128.f), 127.f);
}

static unsigned long long check(float s, uint32_t first, uint64_t stride, uint64_t count) {
  const float y = 1.0f / s;
  unsigned long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (uint64_t i = 0; i < count; ++i) {
    const float x = u2f((uint32_t)(first + i * stride));
    const float t = x / s;
    const float q0 = x * y;
    float q = fmaf(fmaf(-q0, s, x), y, q0);
    if (!(q == q)) q = t;
    const float at = fabsf(t);
    if (at >= 0.125f && at <= 1024.f && f2u(q) != f2u(t)) ++bad;
    if (t == t) {
      if (q8(q, 1) != q8(t, 1)) ++bad;
      if (q8(q, 0) != q8(t, 0)) ++bad;
    }
  }
  return bad;
}

int main(int argc, char** argv) {
  const uint64_t stride = argc > 1 ? strtoull(argv[1], 0, 10) : 4099;
  const uint32_t divisors[] = {0x3c23d70a, 0x3d4ccccd, 0x3f7fffff, 0x3fffffff, 0x3f800000,
                               0x3f800001, 0x3dcccccd, 0x3e99999a, 0x3a83126f, 0x41200000,
                               0x3eaaaaab, 0x3f000001, 0xbd4ccccd, 0x34000000, 0x4b000000,
                               0x3c8efa35, 0x3cf5c28f, 0x3d23d70a, 0x2b800000 /* 2^-40 */,
                               0x53800000 /* 2^40 */};
  unsigned long long bad = 0;
  uint32_t lcg = 12345u;
  for (int round = 0; round < 2; ++round) {
    for (unsigned d = 0; d < sizeof(divisors) / 4; ++d) {
      uint32_t bits = divisors[d];
      if (round == 1) {   /* random significands and exponents within the guarded range */
        lcg = lcg * 1664525u + 1013904223u;
        bits = (lcg & 0x807fffffu) | ((87u + (lcg >> 9) % 81u) << 23);
      }
      const float s = u2f(bits);
      bad += check(s, (uint32_t)d, stride, ((1ull << 32) + stride - 1) / stride);
      /* every x within 2^12 ulps of the ties k + 1/2 of the quantized value, k = -130 .. 130 */
      for (int k = -130; k <= 130; ++k) {
        const float x0 = ((float)k + 0.5f) * s;
        bad += check(s, f2u(x0) - 4096u, 1, 8192);
      }
    }
  }
  printf(bad ? "mismatches: %llu\n" : "ok\n", bad);
  return bad != 0;
}
