/* SPDX-License-Identifier: Apache-2.0 */
/*
 * synth.c -- bit-reproducible synthetic inputs for the tests and the benchmark.
 *
 * A counter-based generator: sample i of stream `seed` depends only on
 * (seed, i), so any slice can be produced independently and in parallel.
 * Normals come from Box-Muller with a logarithm and a cosine built from
 * IEEE + - * / and sqrt only (no libm transcendental is called), so the same
 * bits come out on every machine. Compile with -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>

static inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static inline uint64_t draw(uint64_t seed, uint64_t i) {
  return mix64(mix64(seed * 0xD1342543DE82EF95ull + 0x9E3779B97F4A7C15ull) +
               (i + 1) * 0x9E3779B97F4A7C15ull);
}

/* natural log of u in (0, 1], |error| ~ 1e-16 */
static double det_log(double u) {
  int e;
  double m = frexp(u, &e); /* exact */
  if (m < 0.70710678118654752440) {
    m *= 2.0;
    e -= 1;
  }
  const double s = (m - 1.0) / (m + 1.0), s2 = s * s;
  double p = 1.0 / 25.0;
  for (int k = 23; k >= 1; k -= 2) p = p * s2 + 1.0 / (double)k;
  return (double)e * 0.69314718055994530942 + 2.0 * s * p;
}
/* sin / cos on [0, pi/4] by Taylor series */
static double det_sin(double x) {
  const double x2 = x * x;
  double p = -1.0 / 1307674368000.0; /* -1/15! */
  p = p * x2 + 1.0 / 6227020800.0;
  p = p * x2 - 1.0 / 39916800.0;
  p = p * x2 + 1.0 / 362880.0;
  p = p * x2 - 1.0 / 5040.0;
  p = p * x2 + 1.0 / 120.0;
  p = p * x2 - 1.0 / 6.0;
  p = p * x2 + 1.0;
  return x * p;
}
static double det_cos(double x) {
  const double x2 = x * x;
  double p = 1.0 / 20922789888000.0; /* 1/16! */
  p = p * x2 - 1.0 / 87178291200.0;
  p = p * x2 + 1.0 / 479001600.0;
  p = p * x2 - 1.0 / 3628800.0;
  p = p * x2 + 1.0 / 40320.0;
  p = p * x2 - 1.0 / 720.0;
  p = p * x2 + 1.0 / 24.0;
  p = p * x2 - 1.0 / 2.0;
  p = p * x2 + 1.0;
  return p;
}
/* cos(2*pi*v) for v = k / 2^24 */
static double det_cos2pi(double v) {
  const double q = v * 8.0; /* exact */
  const int oct = (int)q;
  const double f = q - (double)oct;
  const double QPI = 0.78539816339744830962;
  const double a = f * QPI, b = (1.0 - f) * QPI;
  switch (oct & 7) {
  case 0: return det_cos(a);
  case 1: return det_sin(b);
  case 2: return -det_sin(a);
  case 3: return -det_cos(b);
  case 4: return -det_cos(a);
  case 5: return -det_sin(b);
  case 6: return det_sin(a);
  default: return det_cos(b);
  }
}

/* out[i] = float(sigma * N(0,1)), i in [0, n), stream `seed`, starting at sample `first` */
void synth_normal(uint64_t seed, uint64_t first, int64_t n, double sigma, float *out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const uint64_t z = draw(seed, first + (uint64_t)i);
    const double u1 = (double)((z >> 40) + 1) * (1.0 / 16777216.0);    /* (0, 1] */
    const double u2 = (double)((z >> 16) & 0xFFFFFFu) * (1.0 / 16777216.0); /* [0, 1) */
    const double r = sqrt(-2.0 * det_log(u1));
    out[i] = (float)(sigma * (r * det_cos2pi(u2)));
  }
}

/* out[i] uniform integer in [0, bound) */
void synth_uniform_int(uint64_t seed, uint64_t first, int64_t n, int32_t bound, int32_t *out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i)
    out[i] = (int32_t)((draw(seed, first + (uint64_t)i) >> 11) % (uint64_t)bound);
}
