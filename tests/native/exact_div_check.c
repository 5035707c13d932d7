/*
 * Exhaustive check of the three-instruction division the FP8 quantisation kernels use for 16-bit inputs:
 *
 *     r = 1.0f / s            (IEEE, once per row)
 *     q = x * r;  e = fmaf(q, s, -x);  result = fmaf(-e, r, q)        (e = q*s - x exactly: the residual, negated)
 *
 * against the IEEE quotient x / s, for EVERY fp32 significand of s and EVERY significand x of the given width
 * (mant_bits = 7: bfloat16, 10: float16).  Scaling x or s by a power of two scales every intermediate by a power of
 * two, so one binade of each covers all normal-range inputs.  Prints the number of mismatches; exit status 0 iff none.
 * A third argument of 1 checks the plain reciprocal multiply q instead (which must show mismatches: the checker's own
 * sanity test).
 *
 * Build:  gcc -O2 -mfma -ffp-contract=off -fopenmp exact_div_check.c -o exact_div_check -lm
 * Run:    ./exact_div_check 7      (about a second)      ./exact_div_check 10   (ten seconds on 8 cores)
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static inline float bits2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float fast_div(float x, float s, float r) {
  const float q = x * r;
  const float e = fmaf(q, s, -x);
  return fmaf(-e, r, q);
}
/* The zero cases go through separate, non-inlined steps: merged into one expression the host compiler rewrites
 * -(q*s - x) as (-q)*s + x, which loses the sign of a zero residual (the device code pins the two fused operations
 * as written). */
static __attribute__((noinline)) float step_residual(float q, float s, float x) { return fmaf(q, s, -x); }
static __attribute__((noinline)) float step_finish(float e, float r, float q) { return fmaf(-e, r, q); }
static __attribute__((noinline)) float ieee_div_opaque(float x, float s) { return x / s; }

int main(int argc, char** argv) {
  const int mant_bits = argc > 1 ? atoi(argv[1]) : 7;
  const uint32_t stride = argc > 2 ? (uint32_t)atoi(argv[2]) : 1u;      /* > 1: every stride-th significand of s */
  const int naive = argc > 3 ? atoi(argv[3]) : 0;
  if (mant_bits < 1 || mant_bits > 23 || stride < 1) return 2;
  const uint32_t nx = 1u << mant_bits;
  long long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (uint32_t ms = 0; ms < (1u << 23); ms += stride) {
    const volatile float s = bits2f(0x3f800000u | ms);                  /* s in [1, 2) */
    const float r = 1.0f / s;
    for (uint32_t mx = 0; mx < nx; ++mx) {
      const float x = bits2f(0x3f800000u | (mx << (23 - mant_bits)));   /* x in [1, 2): x / s covers (0.5, 2) */
      const float fast = naive ? x * r : fast_div(x, s, r);
      const float ref = x / s;
      if (f2bits(fast) != f2bits(ref)) { ++bad; if (bad < 5) printf("s=%08x x=%08x fast=%08x ref=%08x\n", f2bits(s), f2bits(x), f2bits(fast), f2bits(ref)); }
    }
  }
  /* signed zeros keep their sign (x / s = x for x = +-0), as the quantisers rely on for the code 0x80 */
  for (int neg = 0; neg < 2; ++neg) {
    const float x = neg ? -0.0f : 0.0f, sz = 0.0371f, r = ieee_div_opaque(1.0f, sz), q = x * r;
    const float fast = step_finish(step_residual(q, sz, x), r, q);
    if (f2bits(fast) != f2bits(ieee_div_opaque(x, sz)) || f2bits(fast) != f2bits(x)) {
      ++bad;
      printf("zero case %d: %08x\n", neg, f2bits(fast));
    }
  }
  printf("mant_bits=%d stride=%u mismatches=%lld\n", mant_bits, stride, bad);
  return bad == 0 ? 0 : 1;
}
