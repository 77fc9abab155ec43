/* SPDX-License-Identifier: Apache-2.0 */
/*
 * selfcheck.c -- TEST INFRASTRUCTURE ONLY. Drives every entry point of nntr_oracle.c once on
 * small seeded inputs, with row counts, widths and token counts that reach the leftover-row,
 * partial-block and single-token branches. Built with -fsanitize=address,undefined by
 * `make asan` (oracle/Makefile) so that an out-of-bounds access or undefined operation in
 * the checker itself fails a CPU test instead of skewing a parity result. Checks only what
 * needs no second implementation: round trips, finiteness, and that a one-row product equals
 * the matching row of a product of several rows where the path defines it so.
 */
#include "nntr_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static unsigned long long rng_state = 0x9e3779b97f4a7c15ull;
static float rnd(float scale) {
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  const double u = (double)(rng_state >> 11) / 9007199254740992.0; /* [0, 1) */
  return (float)((u * 2.0 - 1.0) * scale);
}
static float *randv(size_t n, float scale) {
  float *v = (float *)malloc(n * sizeof(float));
  for (size_t i = 0; i < n; ++i) v[i] = rnd(scale);
  return v;
}
static int finite_all(const float *v, size_t n) {
  for (size_t i = 0; i < n; ++i)
    if (!isfinite(v[i])) return 0;
  return 1;
}
#define REQUIRE(c)                                                     \
  do {                                                                 \
    if (!(c)) {                                                        \
      fprintf(stderr, "selfcheck failed: %s (line %d)\n", #c, __LINE__); \
      return 1;                                                        \
    }                                                                  \
  } while (0)

static size_t wbytes(int kind, int n, int k) {
  return kind == 2 ? (size_t)n * (k / 32) * 18 : kind == 12 ? (size_t)n * (k / 256) * 144 : (size_t)n * (k / 256) * 210;
}
static void wquant(int kind, const float *w, void *dst, int n, int k) {
  if (kind == 2) orc_quantize_q4_0(w, dst, n, k);
  else if (kind == 12) orc_quantize_q4_K(w, dst, n, k);
  else orc_quantize_q6_K(w, dst, n, k);
}
static void gemm(int kind, int M, int N, int K, const float *A, const void *W, float *C) {
  if (kind == 2) orc_gemm_q4_0(M, N, K, A, W, C);
  else if (kind == 12) orc_gemm_q4_K(M, N, K, A, W, C);
  else orc_gemm_q6_K(M, N, K, A, W, C);
}

int main(void) {
  const int kinds[3] = {2, 12, 14};
  const int N = 24, K = 512;
  /* half conversions over every bit pattern */
  for (unsigned h = 0; h < 65536; ++h) {
    const float f = orc_fp16_to_fp32((uint16_t)h);
    if (f == f) REQUIRE(orc_fp32_to_fp16(f) == h || (h & 0x7fff) == 0);
  }
  float *w32 = randv((size_t)N * K, 0.05f);
  memset(w32 + K, 0, 256 * sizeof(float)); /* an all-zero super-block */
  float *back = (float *)malloc((size_t)N * K * sizeof(float));
  for (int ki = 0; ki < 3; ++ki) {
    const int kind = kinds[ki];
    const size_t nb = wbytes(kind, N, K);
    unsigned char *q = (unsigned char *)malloc(nb), *x8 = (unsigned char *)malloc(nb), *un = (unsigned char *)malloc(nb);
    wquant(kind, w32, q, N, K);
    if (kind == 2) orc_dequantize_q4_0(q, back, (int64_t)N * K);
    else if (kind == 12) orc_dequantize_q4_K(q, back, (int64_t)N * K);
    else orc_dequantize_q6_K(q, back, (int64_t)N * K);
    REQUIRE(finite_all(back, (size_t)N * K));
    if (kind == 2) {
      REQUIRE(orc_repack_q4_0_x8(x8, q, N, K) == 0 && orc_unpack_q4_0_x8(un, x8, N, K) == 0);
      REQUIRE(memcmp(un, q, nb) == 0);
      REQUIRE(orc_repack_q4_0_x8(x8, q, N - 1, K) != 0); /* rows not a multiple of eight: refused */
    } else if (kind == 12) {
      REQUIRE(orc_repack_q4_K_x8(x8, q, N, K) == 0 && orc_unpack_q4_K_x8(un, x8, N, K) == 0);
      REQUIRE(memcmp(un, q, nb) == 0);
    }
    /* row counts that take only the row path, only the 4-row path, and both */
    const int ms[5] = {1, 3, 4, 7, 9};
    for (int mi = 0; mi < 5; ++mi) {
      const int M = ms[mi];
      float *a = randv((size_t)M * K, 1.0f), *c = (float *)malloc((size_t)M * N * sizeof(float));
      gemm(kind, M, N, K, a, q, c);
      REQUIRE(finite_all(c, (size_t)M * N));
      if (kind != 12 || M < 4) { /* rows are independent wherever the 4-row rule does not apply */
        float *c1 = (float *)malloc((size_t)N * sizeof(float));
        gemm(kind, 1, N, K, a + (size_t)(M - 1) * K, q, c1);
        REQUIRE(memcmp(c1, c + (size_t)(M - 1) * N, (size_t)N * sizeof(float)) == 0);
        free(c1);
      }
      free(a);
      free(c);
    }
    free(q);
    free(x8);
    free(un);
  }
  /* activation quantizers and their round trips */
  {
    float *x = randv(4 * (size_t)K, 3.0f);
    x[5] = 0.f;
    memset(x + K, 0, 256 * sizeof(float));
    unsigned char *r0 = (unsigned char *)calloc(4, (K / 32) * 34), *rk = (unsigned char *)calloc(4, (K / 256) * 292),
                  *rm = (unsigned char *)calloc(4, (K / 256) * 292), *il = (unsigned char *)calloc(4, (K / 256) * 292),
                  *i0 = (unsigned char *)calloc(4, (K / 32) * 34);
    for (int r = 0; r < 4; ++r) {
      orc_quantize_row_q8_0(x + (size_t)r * K, r0 + (size_t)r * (K / 32) * 34, K);
      orc_quantize_row_q8_K(x + (size_t)r * K, rk + (size_t)r * (K / 256) * 292, K);
      orc_quantize_row_q8_K_mat(x + (size_t)r * K, rm + (size_t)r * (K / 256) * 292, K);
    }
    orc_interleave_q8_0x4(r0, i0, K);
    orc_interleave_q8_Kx4(rm, il, K);
    orc_dequantize_q8_0(r0, back, 4 * (int64_t)K);
    for (size_t i = 0; i < 4 * (size_t)K; ++i) REQUIRE(fabsf(back[i] - x[i]) <= 3.0f / 127.f);
    orc_dequantize_q8_K(rk, back, 4 * (int64_t)K);
    for (size_t i = 0; i < 4 * (size_t)K; ++i) REQUIRE(fabsf(back[i] - x[i]) <= 3.0f / 127.f);
    free(x); free(r0); free(rk); free(rm); free(il); free(i0);
  }
  /* swiglu forms */
  {
    const int n = 29; /* ends in the masked step of the vector form */
    float *y = randv(n, 6.0f), *z = randv(n, 2.0f), a[29], b[29], c[29];
    orc_swiglu(n, a, y, z);
    orc_swiglu_x86(n, b, y, z);
    orc_swiglu_alpha_x86(n, c, y, z, 1.702f);
    for (int i = 0; i < n; ++i) REQUIRE(fabsf(a[i] - b[i]) <= 2e-5f * (fabsf(a[i]) + 1.f) && isfinite(c[i]));
    free(y); free(z);
  }
  /* the mixture-of-experts blocks: plain, without renormalisation, GPT-OSS, and the cached layers
   * with one token (row forms only) and with thirteen (4-row groups plus leftovers) */
  {
    const int T = 13, H = 256, I = 256, E = 5, topk = 2;
    const void *gate[5], *up[5], *down[5];
    for (int e = 0; e < E; ++e) {
      float *wg = randv((size_t)I * H, 0.05f), *wu = randv((size_t)I * H, 0.05f), *wd = randv((size_t)H * I, 0.05f);
      void *g = malloc(wbytes(12, I, H)), *u = malloc(wbytes(12, I, H)), *d = malloc(wbytes(12, H, I));
      orc_quantize_q4_K(wg, g, I, H);
      orc_quantize_q4_K(wu, u, I, H);
      orc_quantize_q4_K(wd, d, H, I);
      gate[e] = g, up[e] = u, down[e] = d;
      free(wg); free(wu); free(wd);
    }
    float *x = randv((size_t)T * H, 1.0f), *lg = randv((size_t)T * E, 2.0f);
    float *gb = randv((size_t)E * I, 4.0f), *ub = randv((size_t)E * I, 4.0f), *db = randv((size_t)E * H, 0.3f);
    float *y = (float *)malloc((size_t)T * H * sizeof(float)), *y1 = (float *)malloc((size_t)T * H * sizeof(float));
    int32_t idx[26];
    float wt[26];
    orc_moe_forward(12, 1, T, H, I, E, topk, x, lg, gate, up, down, y, idx, wt);
    REQUIRE(finite_all(y, (size_t)T * H));
    for (int t = 0; t < T; ++t) REQUIRE(fabsf(wt[2 * t] + wt[2 * t + 1] - 1.f) < 1e-5f && idx[2 * t] != idx[2 * t + 1]);
    orc_moe_forward(12, 0, T, H, I, E, topk, x, lg, gate, up, down, y, NULL, NULL);
    orc_moe_forward_q4_K(T, H, I, E, topk, x, lg, gate, up, down, y, NULL, NULL);
    orc_moe_forward_gpt_oss(12, 1, T, H, I, E, topk, x, lg, gate, up, down, gb, ub, db, 1.702f, y, NULL, NULL);
    REQUIRE(finite_all(y, (size_t)T * H));
    orc_moe_forward_cached(12, 0, T, H, I, E, topk, x, lg, gate, up, down, NULL, NULL, NULL, 0.f, 0.f, y, idx, wt);
    orc_moe_forward_cached(12, 1, T, H, I, E, topk, x, lg, gate, up, down, gb, ub, db, 1.702f, 7.0f, y, NULL, NULL);
    REQUIRE(finite_all(y, (size_t)T * H));
    /* one token: the cached Qwen layer evaluates what the per-token layer does */
    orc_moe_forward_cached(12, 0, 1, H, I, E, topk, x, lg, gate, up, down, NULL, NULL, NULL, 0.f, 0.f, y, NULL, NULL);
    orc_moe_forward(12, 1, 1, H, I, E, topk, x, lg, gate, up, down, y1, NULL, NULL);
    REQUIRE(memcmp(y, y1, (size_t)H * sizeof(float)) == 0);
    for (int e = 0; e < E; ++e) {
      free((void *)gate[e]); free((void *)up[e]); free((void *)down[e]);
    }
    free(x); free(lg); free(gb); free(ub); free(db); free(y); free(y1);
  }
  free(w32);
  free(back);
  printf("ORACLE SELFCHECK PASSED\n");
  return 0;
}
