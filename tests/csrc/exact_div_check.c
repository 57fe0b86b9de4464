/* CPU proof-by-search for the division shortcut the quant kernels use.
 *
 * The kernels replace the IEEE divide x / y by
 *     r  = 1.0f / y            (correctly rounded, once per group)
 *     q0 = x * r
 *     e  = fmaf(-q0, y, x)     (exact remainder)
 *     q  = fmaf(e, r, q0)
 * which is the correctly rounded quotient whenever r is the correctly rounded
 * reciprocal and no intermediate under/overflows (Markstein's theorem).  This
 * program searches for a counter-example over the inputs the path produces:
 * every bf16 and fp16 numerator against scales y = amax / max8, plus random
 * fp32 pairs.  It also checks  amax / max8  computed the same way with the
 * host-rounded reciprocal of max8.  Returns the number of mismatches.
 *
 * Quotients below 2^-11 are exempt: there the remainder can underflow, and every
 * such quotient encodes to the 8-bit code 0 (the first rounding boundary of
 * e4m3fn is 2^-10, of int8 is 0.5), so a last-bit difference cannot reach a code. */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float fast_div(float x, float y, float r) {
  float q0 = x * r;
  float e = fmaf(-q0, y, x);
  return fmaf(e, r, q0);
}

static inline int differs(float want, float got) {
  if (fabsf(want) < 0x1p-11f && fabsf(got) < 0x1p-11f) return 0;
  uint32_t a, b; memcpy(&a, &want, 4); memcpy(&b, &got, 4); return a != b;
}

static inline uint32_t bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float from_bits(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static inline uint64_t rng(void) {
  rng_state ^= rng_state << 13; rng_state ^= rng_state >> 7; rng_state ^= rng_state << 17;
  return rng_state;
}

/* numerators: all finite bf16 (kind 0) or fp16 (kind 1) values with |x| <= amax */
int64_t check_16bit_numerators(int kind, float max8, int64_t n_scales) {
  int64_t bad = 0;
  float rmax = 1.0f / max8;
  for (int64_t t = 0; t < n_scales; ++t) {
    /* amax drawn from the same 16-bit format, normal range */
    float amax;
    for (;;) {
      uint16_t h = (uint16_t)(rng() & 0x7fff);
      if (kind == 0) amax = from_bits((uint32_t)h << 16);
      else { int e = (h >> 10) & 0x1f; uint32_t m = h & 0x3ff; if (e == 0 || e == 31) continue;
             amax = from_bits(((uint32_t)(e + 112) << 23) | (m << 13)); }
      if (isfinite(amax) && amax >= 1e-10f && amax < 1e30f) break;
    }
    float y = amax / max8;
    if (bits(fast_div(amax, max8, rmax)) != bits(y)) ++bad;
    float r = 1.0f / y;
    for (uint32_t h = 0; h < 0x8000; ++h) {
      float x;
      if (kind == 0) x = from_bits(h << 16);
      else { int e = (h >> 10) & 0x1f; uint32_t m = h & 0x3ff; if (e == 31) continue;
             if (e == 0) x = (float)m * 5.9604644775390625e-08f;
             else x = from_bits(((uint32_t)(e + 112) << 23) | (m << 13)); }
      if (!(x <= amax)) continue;
      float want = x / y;
      float got = fast_div(x, y, r);
      if (differs(want, got)) ++bad;
    }
  }
  return bad;
}

int64_t check_random_fp32(float max8, int64_t n) {
  int64_t bad = 0;
  float rmax = 1.0f / max8;
  for (int64_t t = 0; t < n; ++t) {
    uint64_t z = rng();
    /* amax in [2^-30, 2^30), x = amax * u with |u| <= 1 in a 2^40 dynamic range */
    float amax = from_bits((uint32_t)(((z >> 40) % 60 + 97) << 23) | (uint32_t)(z & 0x7fffff));
    float y = amax / max8;
    if (bits(fast_div(amax, max8, rmax)) != bits(y)) ++bad;
    float r = 1.0f / y;
    for (int j = 0; j < 16; ++j) {
      uint64_t w = rng();
      float x = from_bits((uint32_t)(((w >> 40) % 40 + 87) << 23) | (uint32_t)(w & 0x7fffff));
      x = x * amax; if (x > amax) x = amax;
      float want = x / y, got = fast_div(x, y, r);
      if (differs(want, got)) ++bad;
    }
  }
  return bad;
}
