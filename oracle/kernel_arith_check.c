/*
 * CPU models of two arithmetic shortcuts the HIP rotate+quantize kernel takes, so that tests can
 * check them against the plain IEEE operations over far more operands than a GPU test compares
 * codes for.  TEST INFRASTRUCTURE ONLY: nothing shipped links or loads this file.
 *
 *   oqk_division_mismatches   x / d as  q = fma(x, rh, x * rl);  q' = fma(fma(-q, d, x), rh, q)
 *                             with rh = RN(1 / d), rl = RN(fma(-d, rh, 1) * rh)
 *                             (orbitquant_amd/csrc/rotate_quantize_fast.h, divide_fast), for the
 *                             operand ranges the kernel admits: 2^-80 <= |x| or x == 0, 2^-80 <= d <= 2^20,
 *                             |x| <= d * 2^9 (a value never exceeds the norm of its row)
 *   oqk_fold_threshold        the largest float t with RN(t * c) <= b, by bisection over the
 *                             ordered floats (rotate_quantize_fast.hip, rotate_plan_build_kernel)
 *
 * Build: gcc -O2 -march=x86-64-v3 -ffp-contract=off -fopenmp -shared -fPIC   (fmaf is the hardware FMA)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static uint64_t next_random(uint64_t *s) {  /* splitmix64 */
  uint64_t z = (*s += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}
static float from_bits(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float divide_fast(float x, float d, float rh, float rl) {
  const float q = fmaf(x, rh, x * rl);
  return fmaf(fmaf(-q, d, x), rh, q);
}

/* mode 0: x has a bf16 significand (8 bits), 1: fp16 significand (11 bits), 2: any fp32 significand;
 * + 16: the control, a sequence that is NOT exact (the first quotient without its correction),
 * which this check must catch.  Every fourth denominator has a special significand (all ones, one, all ones but the last ...). */
int64_t oqk_division_mismatches(int64_t pairs, uint64_t seed, int mode, float *first_x, float *first_d) {
  int64_t bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (int64_t chunk = 0; chunk < 1024; ++chunk) {
    uint64_t s = seed * 1024 + (uint64_t)chunk;
    for (int64_t i = chunk; i < pairs; i += 1024) {
      const uint64_t r = next_random(&s), r2 = next_random(&s);
      uint32_t dm = (uint32_t)(r & 0x7fffff);
      switch ((r >> 60) & 15) {
        case 0: dm = 0x7fffff; break;
        case 1: dm = 0; break;
        case 2: dm = 0x7ffffe; break;
        case 3: dm = 1; break;
        default: break;
      }
      const int de = -80 + (int)((r >> 24) % 101);             /* 2^-80 .. 2^20 */
      const float d = from_bits(((uint32_t)(de + 127) << 23) | dm);
      uint32_t xm = (uint32_t)(r2 & 0x7fffff);
      if ((mode & 7) == 0) xm &= 0x7f0000;
      else if ((mode & 7) == 1) xm &= 0x7fe000;
      int xe = de + 9 - (int)((r2 >> 24) % 64);                /* |x| <= d * 2^9, down to d * 2^-54 */
      if (xe < -80) xe = -80;
      const float x = from_bits(((uint32_t)(r2 >> 63) << 31) | ((uint32_t)(xe + 127) << 23) | xm);
      const float rh = 1.0f / d;
      const float rl = fmaf(-d, rh, 1.0f) * rh;
      const float want = x / d, got = (mode & 16) ? fmaf(x, rh, x * rl) : divide_fast(x, d, rh, rl);
      if (to_bits(want) != to_bits(got)) {
        if (bad == 0 && first_x != 0) { *first_x = x; *first_d = d; }
        ++bad;
      }
    }
  }
  return bad;
}

static uint32_t float_to_ordered(float f) { const uint32_t u = to_bits(f); return (u & 0x80000000u) ? ~u : (u | 0x80000000u); }
static float ordered_to_float(uint32_t o) { return from_bits((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o); }

float oqk_fold_threshold(float b, float c) {
  if (b != b) return b;
  uint32_t lo = float_to_ordered(-INFINITY), hi = float_to_ordered(INFINITY);
  if (INFINITY * c <= b) return INFINITY;
  while (hi - lo > 1) {
    const uint32_t mid = lo + (hi - lo) / 2;
    if (ordered_to_float(mid) * c <= b) lo = mid; else hi = mid;
  }
  return ordered_to_float(lo);
}

/* (b < RN(y * c)) == (t < y) for the `span` floats on either side of t and a few far ones; returns the mismatches. */
int64_t oqk_fold_mismatches(float b, float c, int span) {
  const float t = oqk_fold_threshold(b, c);
  int64_t bad = 0;
  const uint32_t o = float_to_ordered(t);
  for (int k = -span; k <= span; ++k) {
    const uint32_t ok = o + (uint32_t)k;
    const float y = ordered_to_float(ok);
    if (y != y) continue;
    if ((b < y * c) != (t < y)) ++bad;
  }
  const float far[6] = {-INFINITY, -3.0e38f, -0.0f, 0.0f, 3.0e38f, INFINITY};
  for (int k = 0; k < 6; ++k)
    if ((b < far[k] * c) != (t < far[k])) ++bad;
  return bad;
}
