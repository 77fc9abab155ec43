/* SPDX-License-Identifier: Apache-2.0 */
/*
 * nntr_oracle.c -- TEST INFRASTRUCTURE ONLY (see nntr_oracle.h).
 *
 * Plain-C restatement of the reference CPU arithmetic for the quantized matmul
 * path. Compile with -ffp-contract=off: every fused multiply-add that the
 * reference performs (explicit intrinsics in its AVX2 kernels, or contractions
 * GCC applies to its scalar code under the reference's flags) is written out as
 * fmaf() here, so the result does not depend on this file's compiler.
 *
 * GI   = nntrainer/tensor/cpu_backend/ggml_interface
 * IMPL = GI/nntr_ggml_impl
 */
#include "nntr_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <xmmintrin.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* small helpers                                                              */
/* ------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline int imin(int a, int b) { return a < b ? a : b; }
static inline int imax(int a, int b) { return a > b ? a : b; }

#define ROUND_MAGIC 12582912.f /* 1.5 * 2^23 */

/* Integer nearest to v (ties to even) read out of the mantissa of v + 1.5*2^23.
 * IMPL/nntr_ggml_impl_common.h:158-164. `biased` is the already-added value. */
static inline int magic_to_int(float biased) {
  return (int)(f32_bits(biased) & 0x007fffffu) - 0x00400000;
}
/* nearest_int of a plain value (sum rounded once). */
static inline int nearest_int_plain(float v) { return magic_to_int(v + ROUND_MAGIC); }
/* nearest_int(a*b) as GCC emits it under -mfma: the product is never rounded on
 * its own, a*b + magic is one fused operation. */
static inline int nearest_int_prod(float a, float b) {
  return magic_to_int(fmaf(a, b, ROUND_MAGIC));
}

/* ------------------------------------------------------------------------- */
/* binary16                                                                   */
/* ------------------------------------------------------------------------- */

/* IMPL/nntr_ggml_impl_fp16_fp32.cpp:69-79 (F16C _cvtsh_ss) -- exact widening. */
float orc_fp16_to_fp32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1fu;
  const uint32_t m = h & 0x3ffu;
  if (e == 0) {
    /* zero / subnormal: m * 2^-24, exact in binary32 */
    float v = (float)m * 0x1p-24f;
    return bits_f32(f32_bits(v) | sign);
  }
  if (e == 31)
    return bits_f32(sign | 0x7f800000u | (m << 13) | (m ? 0x00400000u : 0));
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* IMPL/nntr_ggml_impl_fp16_fp32.cpp:69-79 (F16C _cvtss_sh(x, 0)) -- round to
 * nearest even, subnormals kept, overflow to infinity. */
uint16_t orc_fp32_to_fp16(float f) {
  uint32_t x = f32_bits(f);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) /* NaN: quiet, keep top payload bits */
    return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu));
  if (x >= 0x477ff000u) /* >= 65520 rounds to infinity */
    return (uint16_t)(sign | 0x7c00u);
  if (x < 0x38800000u) {
    /* below 2^-14: result is a multiple of 2^-24; adding 0.5f makes the fp32
     * adder do the round-to-nearest-even at exactly that grid */
    float v = bits_f32(x) + 0.5f;
    return (uint16_t)(sign | (f32_bits(v) - 0x3f000000u));
  }
  const uint32_t odd = (x >> 13) & 1u;
  x += 0xc8000fffu + odd; /* rebias exponent by -112, add rounding increment */
  return (uint16_t)(sign | (x >> 13));
}

/* ------------------------------------------------------------------------- */
/* block views                                                                */
/* ------------------------------------------------------------------------- */

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline void wr16(uint8_t *p, uint16_t v) {
  p[0] = (uint8_t)(v & 0xff);
  p[1] = (uint8_t)(v >> 8);
}

/* Q4_K: the 12 scale bytes hold eight 6-bit scales and eight 6-bit mins.
 * IMPL/nntr_ggml_impl_quant.cpp:368-378. */
static inline void q4k_scale_min(int j, const uint8_t *s, int *sc, int *mn) {
  if (j < 4) {
    *sc = s[j] & 63;
    *mn = s[j + 4] & 63;
  } else {
    *sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
    *mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
  }
}
static inline void q4k_put_scale_min(int j, uint8_t *s, int sc, int mn) {
  /* inverse of the above; s must start zeroed for j >= 4 to OR into j-4, j */
  if (j < 4) {
    s[j] = (uint8_t)sc;
    s[j + 4] = (uint8_t)mn;
  } else {
    s[j + 4] = (uint8_t)((sc & 0x0f) | ((mn & 0x0f) << 4));
    s[j - 4] |= (uint8_t)((sc >> 4) << 6);
    s[j] |= (uint8_t)((mn >> 4) << 6);
  }
}

/* Q4_K element e (0..255) of a block: sub-block j = e/32 lives in the 32-byte
 * chunk j/2, low nibbles for even j, high nibbles for odd j. */
static inline int q4k_nibble(const uint8_t *qs, int e) {
  const int j = e >> 5, i = e & 31;
  const uint8_t b = qs[(j >> 1) * 32 + i];
  return (j & 1) ? (b >> 4) : (b & 0x0f);
}

/* Q6_K element e (0..255): value in 0..63 (IMPL/nntr_ggml_impl_quant.cpp:1291-1325). */
static inline int q6k_value(const uint8_t *ql, const uint8_t *qh, int e) {
  const int half = e >> 7, r = e & 127, grp = r >> 5, l = r & 31;
  const uint8_t lo = ql[half * 64 + (grp & 1) * 32 + l];
  const int nib = (grp & 2) ? (lo >> 4) : (lo & 0x0f);
  const int hi = (qh[half * 32 + l] >> (2 * grp)) & 3;
  return nib | (hi << 4);
}

/* ------------------------------------------------------------------------- */
/* weight quantizers                                                          */
/* ------------------------------------------------------------------------- */

/* IMPL/nntr_ggml_impl_quant.cpp:382-418. d = (signed max-abs)/-8, quants are
 * truncations of x/d + 8.5 (the multiply-add is fused in the reference build). */
void orc_quantize_q4_0(const float *src, void *dst, int64_t nrow, int64_t k) {
  const int64_t nb = nrow * k / 32;
  uint8_t *out = (uint8_t *)dst;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nb; ++b) {
    const float *x = src + b * 32;
    uint8_t *y = out + b * ORC_Q4_0_BYTES;
    float amax = 0.f, vmax = 0.f;
    for (int j = 0; j < 32; ++j) {
      const float a = fabsf(x[j]);
      if (amax < a) {
        amax = a;
        vmax = x[j];
      }
    }
    const float d = vmax / -8;
    const float id = d ? 1.0f / d : 0.0f;
    wr16(y, orc_fp32_to_fp16(d));
    for (int j = 0; j < 16; ++j) {
      const int lo = imin(15, (int8_t)fmaf(x[j], id, 8.5f));
      const int hi = imin(15, (int8_t)fmaf(x[j + 16], id, 8.5f));
      y[2 + j] = (uint8_t)(lo | (hi << 4));
    }
  }
}

/* Scale/min search for one 32-element Q4_K sub-block.
 * IMPL/nntr_ggml_impl_quant.cpp:115-200 with n=32, nmax=15, rmin=-1,
 * rdelta=0.1, nstep=20, squared-error metric. Returns scale, *neg_min = -min. */
static float q4k_fit_subblock(const float *x, const float *w, uint8_t *L, float *neg_min) {
  float lo = x[0], hi = x[0];
  float sum_w = w[0];
  float sum_x = sum_w * x[0];
  for (int i = 1; i < 32; ++i) {
    if (x[i] < lo) lo = x[i];
    if (x[i] > hi) hi = x[i];
    sum_w += w[i];
    sum_x = fmaf(w[i], x[i], sum_x);
  }
  if (lo > 0) lo = 0;
  if (hi == lo) {
    memset(L, 0, 32);
    *neg_min = -lo;
    return 0.f;
  }
  float iscale = 15 / (hi - lo);
  float scale = 1 / iscale;
  float best = 0;
  for (int i = 0; i < 32; ++i) {
    const int l = nearest_int_prod(iscale, x[i] - lo);
    L[i] = (uint8_t)imax(0, imin(15, l));
    float diff = fmaf(scale, (float)L[i], lo) - x[i];
    diff = diff * diff;
    best = fmaf(w[i], diff, best);
  }
  uint8_t Laux[32];
  for (int is = 0; is <= 20; ++is) {
    iscale = (fmaf(0.1f, (float)is, -1.f) + 15) / (hi - lo);
    float sum_l = 0, sum_l2 = 0, sum_xl = 0;
    for (int i = 0; i < 32; ++i) {
      int l = nearest_int_prod(iscale, x[i] - lo);
      l = imax(0, imin(15, l));
      Laux[i] = (uint8_t)l;
      const float wl = w[i] * (float)l;
      sum_l += wl;
      sum_l2 = fmaf(wl, (float)l, sum_l2);
      sum_xl = fmaf(wl, x[i], sum_xl);
    }
    const float D = fmaf(sum_w, sum_l2, -(sum_l * sum_l));
    if (D > 0) {
      float this_scale = fmaf(-sum_x, sum_l, sum_w * sum_xl) / D;
      float this_min = fmaf(sum_l2, sum_x, -(sum_l * sum_xl)) / D;
      if (this_min > 0) {
        this_min = 0;
        this_scale = sum_xl / sum_l2;
      }
      float err = 0;
      for (int i = 0; i < 32; ++i) {
        float diff = fmaf(this_scale, (float)Laux[i], this_min) - x[i];
        diff = diff * diff;
        err = fmaf(w[i], diff, err);
      }
      if (err < best) {
        memcpy(L, Laux, 32);
        best = err;
        scale = this_scale;
        lo = this_min;
      }
    }
  }
  *neg_min = -lo;
  return scale;
}

/* IMPL/nntr_ggml_impl_quant.cpp:901-979. */
void orc_quantize_q4_K(const float *src, void *dst, int64_t nrow, int64_t k) {
  const int64_t nb = nrow * k / ORC_QK_K;
  uint8_t *out = (uint8_t *)dst;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nb; ++b) {
    const float *x = src + b * ORC_QK_K;
    uint8_t *y = out + b * ORC_Q4_K_BYTES;
    uint8_t L[ORC_QK_K];
    float w[32], mins[8], scales[8];
    float max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; ++j) {
      const float *xs = x + 32 * j;
      float sum_x2 = 0;
      for (int l = 0; l < 32; ++l) sum_x2 = fmaf(xs[l], xs[l], sum_x2);
      const float av_x = sqrtf(sum_x2 / 32);
      for (int l = 0; l < 32; ++l) w[l] = av_x + fabsf(xs[l]);
      scales[j] = q4k_fit_subblock(xs, w, L + 32 * j, &mins[j]);
      if (scales[j] > max_scale) max_scale = scales[j];
      if (mins[j] > max_min) max_min = mins[j];
    }
    const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    uint8_t *sc = y + 4;
    memset(sc, 0, 12);
    for (int j = 0; j < 8; ++j) {
      int ls = (uint8_t)nearest_int_prod(inv_scale, scales[j]);
      int lm = (uint8_t)nearest_int_prod(inv_min, mins[j]);
      ls = imin(63, ls);
      lm = imin(63, lm);
      q4k_put_scale_min(j, sc, ls, lm);
    }
    const uint16_t hd = orc_fp32_to_fp16(max_scale / 63.f);
    const uint16_t hm = orc_fp32_to_fp16(max_min / 63.f);
    wr16(y, hd);
    wr16(y + 2, hm);
    const float fd = orc_fp16_to_fp32(hd), fm = orc_fp16_to_fp32(hm);
    for (int j = 0; j < 8; ++j) {
      int s, m;
      q4k_scale_min(j, sc, &s, &m);
      const float d = fd * (float)s;
      if (!d) continue;
      const float dm = fm * (float)m;
      for (int i = 0; i < 32; ++i) {
        const int l = nearest_int_plain((x[32 * j + i] + dm) / d);
        L[32 * j + i] = (uint8_t)imax(0, imin(15, l));
      }
    }
    uint8_t *q = y + 16;
    for (int c = 0; c < 4; ++c)
      for (int l = 0; l < 32; ++l)
        q[32 * c + l] = (uint8_t)(L[64 * c + l] | (L[64 * c + 32 + l] << 4));
  }
}

/* Symmetric scale search for one 16-element Q6_K group.
 * IMPL/nntr_ggml_impl_quant.cpp:32-113 with n=16, nmax=32, rmse_type=1, no
 * importance weights (weight of element i is x[i]^2). */
static float q6k_fit_group(const float *x, int8_t *L) {
  float vmax = 0, amax = 0;
  for (int i = 0; i < 16; ++i) {
    const float a = fabsf(x[i]);
    if (a > amax) {
      amax = a;
      vmax = x[i];
    }
  }
  if (amax < 1e-15f) {
    memset(L, 0, 16);
    return 0.f;
  }
  float iscale = -32 / vmax;
  float sumlx = 0, suml2 = 0;
  for (int i = 0; i < 16; ++i) {
    int l = nearest_int_prod(iscale, x[i]);
    l = imax(-32, imin(31, l));
    L[i] = (int8_t)(l + 32);
    const float w = x[i] * x[i];
    sumlx = fmaf(w * x[i], (float)l, sumlx);
    suml2 = fmaf(w * (float)l, (float)l, suml2);
  }
  float scale = suml2 ? sumlx / suml2 : 0.0f;
  float best = scale * sumlx;
  for (int is = -9; is <= 9; ++is) {
    if (is == 0) continue;
    iscale = -fmaf(0.1f, (float)is, 32.f) / vmax;
    sumlx = suml2 = 0;
    for (int i = 0; i < 16; ++i) {
      int l = nearest_int_prod(iscale, x[i]);
      l = imax(-32, imin(31, l));
      const float w = x[i] * x[i];
      sumlx = fmaf(w * x[i], (float)l, sumlx);
      suml2 = fmaf(w * (float)l, (float)l, suml2);
    }
    if (suml2 > 0 && sumlx * sumlx > best * suml2) {
      for (int i = 0; i < 16; ++i) {
        const int l = nearest_int_prod(iscale, x[i]);
        L[i] = (int8_t)(32 + imax(-32, imin(31, l)));
      }
      scale = sumlx / suml2;
      best = scale * sumlx;
    }
  }
  return scale;
}

/* IMPL/nntr_ggml_impl_quant.cpp:1116-1186. */
void orc_quantize_q6_K(const float *src, void *dst, int64_t nrow, int64_t k) {
  const int64_t nb = nrow * k / ORC_QK_K;
  uint8_t *out = (uint8_t *)dst;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < nb; ++b) {
    const float *x = src + b * ORC_QK_K;
    uint8_t *y = out + b * ORC_Q6_K_BYTES;
    uint8_t *ql = y, *qh = y + 128;
    int8_t *sc = (int8_t *)(y + 192);
    int8_t L[ORC_QK_K];
    float scales[16];
    float max_scale = 0, max_abs = 0;
    for (int g = 0; g < 16; ++g) {
      scales[g] = q6k_fit_group(x + 16 * g, L + 16 * g);
      const float a = fabsf(scales[g]);
      if (a > max_abs) {
        max_abs = a;
        max_scale = scales[g];
      }
    }
    if (max_abs < 1e-15f) {
      memset(y, 0, ORC_Q6_K_BYTES);
      continue;
    }
    const float iscale = -128.f / max_scale;
    const uint16_t hd = orc_fp32_to_fp16(1 / iscale);
    wr16(y + 208, hd);
    for (int g = 0; g < 16; ++g)
      sc[g] = (int8_t)imin(127, nearest_int_prod(iscale, scales[g]));
    const float fd = orc_fp16_to_fp32(hd);
    for (int g = 0; g < 16; ++g) {
      const float d = fd * (float)sc[g];
      if (!d) continue;
      for (int i = 0; i < 16; ++i) {
        int l = nearest_int_plain(x[16 * g + i] / d);
        l = imax(-32, imin(31, l));
        L[16 * g + i] = (int8_t)(l + 32);
      }
    }
    for (int half = 0; half < 2; ++half) {
      const int8_t *Lh = L + 128 * half;
      for (int l = 0; l < 32; ++l) {
        const int q1 = Lh[l] & 0xf, q2 = Lh[l + 32] & 0xf;
        const int q3 = Lh[l + 64] & 0xf, q4 = Lh[l + 96] & 0xf;
        ql[64 * half + l] = (uint8_t)(q1 | (q3 << 4));
        ql[64 * half + 32 + l] = (uint8_t)(q2 | (q4 << 4));
        qh[32 * half + l] = (uint8_t)((Lh[l] >> 4) | ((Lh[l + 32] >> 4) << 2) |
                                      ((Lh[l + 64] >> 4) << 4) | ((Lh[l + 96] >> 4) << 6));
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* dequantizers                                                               */
/* ------------------------------------------------------------------------- */

/* IMPL/nntr_ggml_impl_quant.cpp:469-488. */
void orc_dequantize_q4_0(const void *blocks, float *y, int64_t n) {
  const uint8_t *p = (const uint8_t *)blocks;
  for (int64_t b = 0; b < n / 32; ++b, p += ORC_Q4_0_BYTES, y += 32) {
    const float d = orc_fp16_to_fp32(rd16(p));
    for (int j = 0; j < 16; ++j) {
      y[j] = (float)((p[2 + j] & 0x0f) - 8) * d;
      y[j + 16] = (float)((p[2 + j] >> 4) - 8) * d;
    }
  }
}

/* IMPL/nntr_ggml_impl_quant.cpp:1079-1108. */
void orc_dequantize_q4_K(const void *blocks, float *y, int64_t n) {
  const uint8_t *p = (const uint8_t *)blocks;
  for (int64_t b = 0; b < n / ORC_QK_K; ++b, p += ORC_Q4_K_BYTES, y += ORC_QK_K) {
    const float d = orc_fp16_to_fp32(rd16(p));
    const float dmin = orc_fp16_to_fp32(rd16(p + 2));
    for (int j = 0; j < 8; ++j) {
      int s, m;
      q4k_scale_min(j, p + 4, &s, &m);
      const float dj = d * (float)s, mj = dmin * (float)m;
      for (int i = 0; i < 32; ++i)
        y[32 * j + i] = dj * (float)q4k_nibble(p + 16, 32 * j + i) - mj;
    }
  }
}

/* IMPL/nntr_ggml_impl_quant.cpp:1291-1325. */
void orc_dequantize_q6_K(const void *blocks, float *y, int64_t n) {
  const uint8_t *p = (const uint8_t *)blocks;
  for (int64_t b = 0; b < n / ORC_QK_K; ++b, p += ORC_Q6_K_BYTES, y += ORC_QK_K) {
    const float d = orc_fp16_to_fp32(rd16(p + 208));
    const int8_t *sc = (const int8_t *)(p + 192);
    for (int e = 0; e < ORC_QK_K; ++e)
      y[e] = d * (float)sc[e >> 4] * (float)(int8_t)(q6k_value(p, p + 128, e) - 32);
  }
}

/* IMPL/nntr_ggml_impl_quant.cpp:876-891. */
void orc_dequantize_q8_0(const void *blocks, float *y, int64_t n) {
  const uint8_t *p = (const uint8_t *)blocks;
  for (int64_t b = 0; b < n / 32; ++b, p += ORC_Q8_0_BYTES, y += 32) {
    const float d = orc_fp16_to_fp32(rd16(p));
    for (int j = 0; j < 32; ++j) y[j] = (float)(int8_t)p[2 + j] * d;
  }
}

/* IMPL/nntr_ggml_impl_quant.cpp:1461-1471. */
void orc_dequantize_q8_K(const void *blocks, float *y, int64_t n) {
  const uint8_t *p = (const uint8_t *)blocks;
  for (int64_t b = 0; b < n / ORC_QK_K; ++b, p += ORC_Q8_K_BYTES, y += ORC_QK_K) {
    float d;
    memcpy(&d, p, 4);
    for (int j = 0; j < ORC_QK_K; ++j) y[j] = d * (float)(int8_t)p[4 + j];
  }
}

/* ------------------------------------------------------------------------- */
/* x8 interleave                                                              */
/* ------------------------------------------------------------------------- */

/* IMPL/nntr_ggml_impl.cpp:8056-8079, 8189-8216: 8 rows' blocks at the same K
 * position become one 144-byte group {d[8], qs[128]}; qs is the 8 rows' 16 quant
 * bytes taken 8 bytes at a time round-robin over rows, every nibble XOR 8. */
int orc_repack_q4_0_x8(void *dst, const void *src, int64_t nrow, int64_t k) {
  if (nrow % 8 || k % 8) return -1;
  const int64_t nb = k / 32;
  const uint8_t *s = (const uint8_t *)src;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t r0 = 0; r0 < nrow; r0 += 8)
    for (int64_t b = 0; b < nb; ++b, d += 144)
      for (int r = 0; r < 8; ++r) {
        const uint8_t *blk = s + ((r0 + r) * nb + b) * ORC_Q4_0_BYTES;
        d[2 * r] = blk[0];
        d[2 * r + 1] = blk[1];
        for (int half = 0; half < 2; ++half)
          for (int i = 0; i < 8; ++i)
            d[16 + half * 64 + r * 8 + i] = blk[2 + half * 8 + i] ^ 0x88;
      }
  return 0;
}

int orc_unpack_q4_0_x8(void *dst, const void *src, int64_t nrow, int64_t k) {
  if (nrow % 8 || k % 8) return -1;
  const int64_t nb = k / 32;
  const uint8_t *s = (const uint8_t *)src;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t r0 = 0; r0 < nrow; r0 += 8)
    for (int64_t b = 0; b < nb; ++b, s += 144)
      for (int r = 0; r < 8; ++r) {
        uint8_t *blk = d + ((r0 + r) * nb + b) * ORC_Q4_0_BYTES;
        blk[0] = s[2 * r];
        blk[1] = s[2 * r + 1];
        for (int half = 0; half < 2; ++half)
          for (int i = 0; i < 8; ++i)
            blk[2 + half * 8 + i] = s[16 + half * 64 + r * 8 + i] ^ 0x88;
      }
  return 0;
}

/* IMPL/nntr_ggml_impl.cpp:8081-8158, 8218-8245: 8 rows' super-blocks become one
 * 1152-byte group {d[8], dmin[8], scales[96], qs[1024]}. qs: 8-byte round-robin
 * over rows. scales: 8 groups of 12 bytes, group g holding sub-block g's scale
 * and min of each of the 8 rows, packed with the same 6-bit scheme but indexed
 * by row instead of by sub-block. */
int orc_repack_q4_K_x8(void *dst, const void *src, int64_t nrow, int64_t k) {
  if (nrow % 8 || k % 8) return -1;
  const int64_t nb = k / ORC_QK_K;
  const uint8_t *s = (const uint8_t *)src;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t r0 = 0; r0 < nrow; r0 += 8)
    for (int64_t b = 0; b < nb; ++b, d += 1152) {
      memset(d + 32, 0, 96);
      for (int r = 0; r < 8; ++r) {
        const uint8_t *blk = s + ((r0 + r) * nb + b) * ORC_Q4_K_BYTES;
        d[2 * r] = blk[0];
        d[2 * r + 1] = blk[1];
        d[16 + 2 * r] = blk[2];
        d[16 + 2 * r + 1] = blk[3];
        for (int c = 0; c < 16; ++c)
          memcpy(d + 128 + c * 64 + r * 8, blk + 16 + c * 8, 8);
      }
      for (int g = 0; g < 8; ++g)
        for (int r = 0; r < 8; ++r) {
          int sc, mn;
          q4k_scale_min(g, s + ((r0 + r) * nb + b) * ORC_Q4_K_BYTES + 4, &sc, &mn);
          q4k_put_scale_min(r, d + 32 + 12 * g, sc, mn);
        }
    }
  return 0;
}

int orc_unpack_q4_K_x8(void *dst, const void *src, int64_t nrow, int64_t k) {
  if (nrow % 8 || k % 8) return -1;
  const int64_t nb = k / ORC_QK_K;
  const uint8_t *s = (const uint8_t *)src;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t r0 = 0; r0 < nrow; r0 += 8)
    for (int64_t b = 0; b < nb; ++b, s += 1152)
      for (int r = 0; r < 8; ++r) {
        uint8_t *blk = d + ((r0 + r) * nb + b) * ORC_Q4_K_BYTES;
        blk[0] = s[2 * r];
        blk[1] = s[2 * r + 1];
        blk[2] = s[16 + 2 * r];
        blk[3] = s[16 + 2 * r + 1];
        memset(blk + 4, 0, 12);
        for (int g = 0; g < 8; ++g) {
          int sc, mn;
          q4k_scale_min(r, s + 32 + 12 * g, &sc, &mn);
          q4k_put_scale_min(g, blk + 4, sc, mn);
        }
        for (int c = 0; c < 16; ++c)
          memcpy(blk + 16 + c * 8, s + 128 + c * 64 + r * 8, 8);
      }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* activation quantizers                                                      */
/* ------------------------------------------------------------------------- */

/* IMPL/nntr_ggml_impl_quant.cpp:613-701: per 32 values, d = fp16(amax/127),
 * quants = round-to-nearest-even of x * (127/amax), the product rounded to
 * fp32 first (vector multiply, then vector round). */
void orc_quantize_row_q8_0(const float *x, void *y, int64_t k) {
  uint8_t *out = (uint8_t *)y;
  for (int64_t b = 0; b < k / 32; ++b, x += 32, out += ORC_Q8_0_BYTES) {
    float amax = 0.f;
    for (int j = 0; j < 32; ++j) {
      const float a = fabsf(x[j]);
      if (a > amax) amax = a;
    }
    wr16(out, orc_fp32_to_fp16(amax / 127.f));
    const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
    for (int j = 0; j < 32; ++j) {
      const float v = x[j] * id;
      out[2 + j] = (uint8_t)(int8_t)(int)nearbyintf(v);
    }
  }
}

/* IMPL/nntr_ggml_impl_quant.cpp:1334-1374 (reached from :1376-1459 on x86).
 * The sign of the scale follows the FIRST element of maximal magnitude. */
void orc_quantize_row_q8_K(const float *x, void *y, int64_t k) {
  uint8_t *out = (uint8_t *)y;
  for (int64_t b = 0; b < k / ORC_QK_K; ++b, x += ORC_QK_K, out += ORC_Q8_K_BYTES) {
    float vmax = 0, amax = 0;
    for (int j = 0; j < ORC_QK_K; ++j) {
      const float a = fabsf(x[j]);
      if (a > amax) {
        amax = a;
        vmax = x[j];
      }
    }
    int8_t *qs = (int8_t *)(out + 4);
    int16_t bs[16];
    if (!amax) {
      /* the reference writes d and qs only; its callers hand it zeroed memory */
      memset(out, 0, ORC_Q8_K_BYTES);
      continue;
    }
    const float iscale = -127.f / vmax;
    for (int j = 0; j < ORC_QK_K; ++j)
      qs[j] = (int8_t)imin(127, nearest_int_prod(iscale, x[j]));
    for (int g = 0; g < 16; ++g) {
      int s = 0;
      for (int i = 0; i < 16; ++i) s += qs[16 * g + i];
      bs[g] = (int16_t)s;
    }
    const float d = 1 / iscale;
    memcpy(out, &d, 4);
    memcpy(out + 260, bs, 32);
  }
}

/* Per-row content of the 4-row AVX2 quantizer IMPL/nntr_ggml_impl.cpp:7504-7737:
 * scale is negative exactly when some element EQUALS +amax, the product x*iscale
 * is rounded to fp32 and then to the nearest-even integer, saturating to int8. */
void orc_quantize_row_q8_K_mat(const float *x, void *y, int64_t k) {
  uint8_t *out = (uint8_t *)y;
  for (int64_t b = 0; b < k / ORC_QK_K; ++b, x += ORC_QK_K, out += ORC_Q8_K_BYTES) {
    float amax = 0;
    for (int j = 0; j < ORC_QK_K; ++j) {
      const float a = fabsf(x[j]);
      if (a > amax) amax = a;
    }
    int pos_hit = 0;
    for (int j = 0; j < ORC_QK_K; ++j) pos_hit |= (x[j] == amax);
    float iscale = (amax != 0.0f) ? 127.f / amax : 0.0f;
    if (pos_hit) iscale = (amax != 0.0f) ? -127.f / amax : 0.0f;
    const float d = amax ? 1 / iscale : 0;
    int8_t *qs = (int8_t *)(out + 4);
    int16_t bs[16];
    for (int j = 0; j < ORC_QK_K; ++j) {
      const float v = nearbyintf(x[j] * iscale);
      int q = (int)v;
      qs[j] = (int8_t)imax(-128, imin(127, q));
    }
    for (int g = 0; g < 16; ++g) {
      int s = 0;
      for (int i = 0; i < 16; ++i) s += qs[16 * g + i];
      bs[g] = (int16_t)s;
    }
    memcpy(out, &d, 4);
    memcpy(out + 260, bs, 32);
  }
}

/* block_q8_0x4 {d[4]; qs[128]}: quants of 4 rows, 8 bytes at a time round-robin.
 * IMPL/nntr_ggml_impl.cpp:7943-7980. rows4 = 4 canonical rows back to back. */
void orc_interleave_q8_0x4(const void *rows4, void *dst, int64_t k) {
  const int64_t nb = k / 32;
  const uint8_t *s = (const uint8_t *)rows4;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t b = 0; b < nb; ++b, d += 136)
    for (int r = 0; r < 4; ++r) {
      const uint8_t *blk = s + (r * nb + b) * ORC_Q8_0_BYTES;
      d[2 * r] = blk[0];
      d[2 * r + 1] = blk[1];
      for (int c = 0; c < 4; ++c) memcpy(d + 8 + c * 32 + r * 8, blk + 2 + c * 8, 8);
    }
}

/* block_q8_Kx4 {d[4]; qs[1024]; bsums[64]}: quants 8 bytes round-robin; the sum
 * of 16-element group g of row r sits at (g/4)*16 + r*4 + g%4.
 * IMPL/nntr_ggml_impl.cpp:7742-7784. */
void orc_interleave_q8_Kx4(const void *rows4, void *dst, int64_t k) {
  const int64_t nb = k / ORC_QK_K;
  const uint8_t *s = (const uint8_t *)rows4;
  uint8_t *d = (uint8_t *)dst;
  for (int64_t b = 0; b < nb; ++b, d += 1168)
    for (int r = 0; r < 4; ++r) {
      const uint8_t *blk = s + (r * nb + b) * ORC_Q8_K_BYTES;
      memcpy(d + 4 * r, blk, 4);
      for (int c = 0; c < 32; ++c) memcpy(d + 16 + c * 32 + r * 8, blk + 4 + c * 8, 8);
      for (int g = 0; g < 16; ++g)
        memcpy(d + 16 + 1024 + 2 * ((g / 4) * 16 + r * 4 + g % 4), blk + 260 + 2 * g, 2);
    }
}

/* ------------------------------------------------------------------------- */
/* block-dot matmuls                                                          */
/* ------------------------------------------------------------------------- */

/* One output element, Q4_0 x Q8_0: per 32-block an exact int32 dot, then
 * acc = fma(float(isum), dw*da, acc), blocks ascending (GEMV and GEMM alike).
 * IMPL/nntr_ggml_impl.cpp:9676-9752, 2878-2901. */
static float dot_q4_0_q8_0(const uint8_t *w, const uint8_t *a, int nb) {
  float acc = 0.f;
  for (int b = 0; b < nb; ++b, w += ORC_Q4_0_BYTES, a += ORC_Q8_0_BYTES) {
    const int8_t *q8 = (const int8_t *)(a + 2);
    int isum = 0;
    for (int j = 0; j < 16; ++j) {
      isum += ((w[2 + j] & 0x0f) - 8) * q8[j];
      isum += ((w[2 + j] >> 4) - 8) * q8[j + 16];
    }
    const float s = orc_fp16_to_fp32(rd16(w)) * orc_fp16_to_fp32(rd16(a));
    acc = fmaf((float)isum, s, acc);
  }
  return acc;
}

/* One output element, Q4_K x Q8_K. `pairwise` = 0: one fma pair per super-block
 * (GEMV kernel, IMPL/nntr_ggml_impl.cpp:7133-7422); 1: one fma pair per two
 * sub-blocks (GEMM kernel, :6274-6989). Result acc - acc_min. */
static float dot_q4_K_q8_K(const uint8_t *w, const uint8_t *a, int nb, int pairwise) {
  float acc = 0.f, accm = 0.f;
  for (int b = 0; b < nb; ++b, w += ORC_Q4_K_BYTES, a += ORC_Q8_K_BYTES) {
    float da;
    memcpy(&da, a, 4);
    const int8_t *q8 = (const int8_t *)(a + 4);
    int16_t bs[16];
    memcpy(bs, a + 260, 32);
    const float sd = orc_fp16_to_fp32(rd16(w)) * da;
    const float sm = orc_fp16_to_fp32(rd16(w + 2)) * da;
    int I = 0, Im = 0;
    for (int j = 0; j < 8; ++j) {
      int sc, mn;
      q4k_scale_min(j, w + 4, &sc, &mn);
      int dot = 0;
      for (int i = 0; i < 32; ++i) dot += q4k_nibble(w + 16, 32 * j + i) * q8[32 * j + i];
      I += sc * dot;
      Im += mn * (bs[2 * j] + bs[2 * j + 1]);
      if (pairwise && (j & 1)) {
        acc = fmaf((float)I, sd, acc);
        accm = fmaf((float)Im, sm, accm);
        I = Im = 0;
      }
    }
    if (!pairwise) {
      acc = fmaf((float)I, sd, acc);
      accm = fmaf((float)Im, sm, accm);
    }
  }
  return acc - accm;
}

/* One output element, Q6_K x Q8_K: eight fp32 partial accumulators, partial l
 * owning the elements whose index mod 32 lies in [4l, 4l+4); per super-block
 * acc[l] = fma(dA*dW, float(S_l), acc[l]); final pairwise tree of hsum_float_8.
 * IMPL/nntr_ggml_impl.cpp:8602-8695, IMPL/nntr_ggml_impl_utils.h:59-66. */
static float dot_q6_K_q8_K(const uint8_t *w, const uint8_t *a, int nb) {
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int b = 0; b < nb; ++b, w += ORC_Q6_K_BYTES, a += ORC_Q8_K_BYTES) {
    float da;
    memcpy(&da, a, 4);
    const int8_t *q8 = (const int8_t *)(a + 4);
    const int8_t *sc = (const int8_t *)(w + 192);
    const float d = da * orc_fp16_to_fp32(rd16(w + 208));
    int S[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int e = 0; e < ORC_QK_K; ++e)
      S[(e & 31) >> 2] += sc[e >> 4] * (q6k_value(w, w + 128, e) - 32) * q8[e];
    for (int l = 0; l < 8; ++l) acc[l] = fmaf(d, (float)S[l], acc[l]);
  }
  return ((acc[0] + acc[4]) + (acc[2] + acc[6])) + ((acc[1] + acc[5]) + (acc[3] + acc[7]));
}

/* GI/ggml_interface_omp.cpp:303-390. Every row's activation is quantized to
 * Q8_0 (row and 4-row quantizers agree per row), every output is the same chain. */
void orc_gemm_q4_0(int M, int N, int K, const float *A, const void *W, float *C) {
  const int nb = K / 32;
  uint8_t *qa = (uint8_t *)malloc((size_t)M * nb * ORC_Q8_0_BYTES);
  for (int m = 0; m < M; ++m)
    orc_quantize_row_q8_0(A + (size_t)m * K, qa + (size_t)m * nb * ORC_Q8_0_BYTES, K);
  const uint8_t *w = (const uint8_t *)W;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m)
      C[(size_t)m * N + n] = dot_q4_0_q8_0(w + (size_t)n * nb * ORC_Q4_0_BYTES,
                                           qa + (size_t)m * nb * ORC_Q8_0_BYTES, nb);
  free(qa);
}

/* GI/ggml_interface_omp.cpp:404-487. M == 1: row quantizer + GEMV kernel.
 * M > 1: rows [0, 4*(M/4)) use the 4-row quantizer and the GEMM kernel, the
 * remaining 1-3 rows the row quantizer and the GEMV kernel. */
void orc_gemm_q4_K(int M, int N, int K, const float *A, const void *W, float *C) {
  const int nb = K / ORC_QK_K;
  const int M4 = (M == 1) ? 0 : (M / 4) * 4;
  uint8_t *qa = (uint8_t *)calloc((size_t)M * nb, ORC_Q8_K_BYTES);
  for (int m = 0; m < M; ++m) {
    uint8_t *row = qa + (size_t)m * nb * ORC_Q8_K_BYTES;
    if (m < M4)
      orc_quantize_row_q8_K_mat(A + (size_t)m * K, row, K);
    else
      orc_quantize_row_q8_K(A + (size_t)m * K, row, K);
  }
  const uint8_t *w = (const uint8_t *)W;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m)
      C[(size_t)m * N + n] =
        dot_q4_K_q8_K(w + (size_t)n * nb * ORC_Q4_K_BYTES,
                      qa + (size_t)m * nb * ORC_Q8_K_BYTES, nb, m < M4);
  free(qa);
}

/* GI/ggml_interface_omp.cpp:500-566: row quantizer for every row, one vec_dot
 * per output element. */
void orc_gemm_q6_K(int M, int N, int K, const float *A, const void *W, float *C) {
  const int nb = K / ORC_QK_K;
  uint8_t *qa = (uint8_t *)calloc((size_t)M * nb, ORC_Q8_K_BYTES);
  for (int m = 0; m < M; ++m)
    orc_quantize_row_q8_K(A + (size_t)m * K, qa + (size_t)m * nb * ORC_Q8_K_BYTES, K);
  const uint8_t *w = (const uint8_t *)W;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n)
    for (int m = 0; m < M; ++m)
      C[(size_t)m * N + n] = dot_q6_K_q8_K(w + (size_t)n * nb * ORC_Q6_K_BYTES,
                                           qa + (size_t)m * nb * ORC_Q8_K_BYTES, nb);
  free(qa);
}

/* ------------------------------------------------------------------------- */
/* mixture of experts                                                         */
/* ------------------------------------------------------------------------- */

/* M == 1 matmul of one weight format into a caller buffer, serial (called from a
 * parallel loop): the row quantizer and the dot kernel the reference's wrappers use for
 * a single row (GI/ggml_interface_omp.cpp:303-330, 404-431, 500-566).
 * kind: 2 Q4_0, 12 Q4_K, 14 Q6_K (the ggml type ids). */
static size_t moe_row_bytes(int kind, int K) {
  return kind == 2 ? (size_t)(K / 32) * ORC_Q4_0_BYTES
                   : (size_t)(K / ORC_QK_K) * (kind == 12 ? ORC_Q4_K_BYTES : ORC_Q6_K_BYTES);
}
static void gemv_serial(int kind, int N, int K, const float *a, const uint8_t *w, float *c, uint8_t *qa) {
  const size_t rb = moe_row_bytes(kind, K);
  if (kind == 2) {
    const int nb = K / 32;
    orc_quantize_row_q8_0(a, qa, K);
    for (int n = 0; n < N; ++n) c[n] = dot_q4_0_q8_0(w + (size_t)n * rb, qa, nb);
    return;
  }
  const int nb = K / ORC_QK_K;
  memset(qa, 0, (size_t)nb * ORC_Q8_K_BYTES);
  orc_quantize_row_q8_K(a, qa, K);
  for (int n = 0; n < N; ++n)
    c[n] = kind == 12 ? dot_q4_K_q8_K(w + (size_t)n * rb, qa, nb, 0) : dot_q6_K_q8_K(w + (size_t)n * rb, qa, nb);
}

/* Routing shared by every variant of the block: softmax over the E logits, top-k by
 * descending probability (ties to the lower index), weights divided by their sum if
 * renormalize. idx, wt [T x topk]. */
static void moe_route(int renormalize, int T, int E, int topk, const float *logits, int32_t *idx, float *wt) {
  float *p = (float *)malloc(sizeof(float) * (size_t)E);
  char *taken = (char *)malloc((size_t)E);
  for (int t = 0; t < T; ++t) {
    const float *lg = logits + (size_t)t * E;
    float mx = lg[0];
    for (int e = 1; e < E; ++e)
      if (lg[e] > mx) mx = lg[e];
    float sum = 0.f;
    for (int e = 0; e < E; ++e) {
      p[e] = (float)exp((double)(lg[e] - mx));
      sum += p[e];
    }
    for (int e = 0; e < E; ++e) p[e] = p[e] / sum;
    memset(taken, 0, (size_t)E);
    float ksum = 0.f;
    for (int k = 0; k < topk; ++k) {
      int best = -1;
      for (int e = 0; e < E; ++e)
        if (!taken[e] && (best < 0 || p[e] > p[best])) best = e;
      taken[best] = 1;
      idx[t * topk + k] = best;
      wt[t * topk + k] = p[best];
      ksum += p[best];
    }
    if (renormalize)
      for (int k = 0; k < topk; ++k) wt[t * topk + k] = wt[t * topk + k] / ksum;
  }
  free(p);
  free(taken);
}

/* Applications/CausalLM/layers/qwen_moe_layer.cpp:394-503 with :332-392 (renormalize
 * = 1, the incremental path) and :161-259 (renormalize = 0, the forwarding path, which
 * uses the softmax values of the selected experts as they are).
 * Routing: softmax over the E logits (subtract row max, exp, divide by the row
 * sum), top-k by descending probability, weights divided by their sum if renormalize.
 * Expert e, token t (one at a time, M = 1): g = x.Wgate, u = x.Wup,
 * h = (sigmoid(g) * g) * u with sigmoid evaluated in double and cast
 * (nntrainer/layers/acti_func.h:286-288, 400-405), o = h.Wdown, contribution =
 * o * weight. Contributions are added into y in ascending expert order. */
static void moe_forward_impl(int kind, int renormalize, int T, int H, int I, int E, int topk, const float *x,
                             const float *logits, const void *const *gate, const void *const *up,
                             const void *const *down, const float *gate_bias, const float *up_bias,
                             const float *down_bias, int gpt_oss, float alpha, float *y, int32_t *topk_idx,
                             float *topk_w) {
  int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)T * topk);
  float *wt = (float *)malloc(sizeof(float) * (size_t)T * topk);
  moe_route(renormalize, T, E, topk, logits, idx, wt);
  if (topk_idx) memcpy(topk_idx, idx, sizeof(int32_t) * (size_t)T * topk);
  if (topk_w) memcpy(topk_w, wt, sizeof(float) * (size_t)T * topk);

  /* contribution of pair (t, k), computed independently, then combined in
   * ascending expert order per token (adding a zero row is exact, so this is
   * the reference's "sum expert_outputs[e] for e ascending"). */
  float *contrib = (float *)malloc(sizeof(float) * (size_t)T * topk * H);
#pragma omp parallel
  {
    const int kmax = H > I ? H : I;
    uint8_t *qa = (uint8_t *)malloc((size_t)(kmax / 32) * ORC_Q8_0_BYTES + (size_t)(kmax / ORC_QK_K + 1) * ORC_Q8_K_BYTES);
    float *g = (float *)malloc(sizeof(float) * (size_t)I);
    float *u = (float *)malloc(sizeof(float) * (size_t)I);
    float *h = (float *)malloc(sizeof(float) * (size_t)I);
#pragma omp for schedule(dynamic)
    for (int pr = 0; pr < T * topk; ++pr) {
      const int t = pr / topk, e = idx[pr];
      const float *xt = x + (size_t)t * H;
      float *o = contrib + (size_t)pr * H;
      gemv_serial(kind, I, H, xt, (const uint8_t *)gate[e], g, qa);
      gemv_serial(kind, I, H, xt, (const uint8_t *)up[e], u, qa);
      if (gpt_oss) {
        /* gpt_oss_moe_layer.cpp:406-437: biases added to the finished products, one added to
         * up, then swiglu with alpha = (Y / (1 + exp(-alpha Y))) * Z in fp32
         * (fallback_internal.cpp:425-432), Y = gate, Z = up + 1 */
        for (int i = 0; i < I; ++i) {
          const float gi = g[i] + gate_bias[(size_t)e * I + i];
          float ui = u[i] + up_bias[(size_t)e * I + i];
          ui = ui + 1.f;
          h[i] = (gi / (1.f + expf(-alpha * gi))) * ui;
        }
      } else {
        for (int i = 0; i < I; ++i) {
          const float en = (float)exp((double)(-g[i]));
          const float sig = (float)(1.0 / (1.0 + (double)en));
          h[i] = (sig * g[i]) * u[i];
        }
      }
      gemv_serial(kind, H, I, h, (const uint8_t *)down[e], o, qa);
      if (gpt_oss) /* gpt_oss_moe_layer.cpp:441: token_expert_output.add_i(down_bias), then the weight */
        for (int c = 0; c < H; ++c) o[c] = o[c] + down_bias[(size_t)e * H + c];
      for (int c = 0; c < H; ++c) o[c] = o[c] * wt[pr];
    }
    free(qa);
    free(g);
    free(u);
    free(h);
  }
  for (int t = 0; t < T; ++t) {
    float *yt = y + (size_t)t * H;
    for (int c = 0; c < H; ++c) yt[c] = 0.f;
    /* visit this token's experts in ascending expert id */
    for (int e = 0; e < E; ++e)
      for (int k = 0; k < topk; ++k)
        if (idx[t * topk + k] == e) {
          const float *o = contrib + ((size_t)t * topk + k) * H;
          for (int c = 0; c < H; ++c) yt[c] = yt[c] + o[c];
        }
  }
  free(contrib);
  free(idx);
  free(wt);
}

void orc_moe_forward(int kind, int renormalize, int T, int H, int I, int E, int topk, const float *x,
                     const float *logits, const void *const *gate, const void *const *up,
                     const void *const *down, float *y, int32_t *topk_idx, float *topk_w) {
  moe_forward_impl(kind, renormalize, T, H, I, E, topk, x, logits, gate, up, down, NULL, NULL, NULL, 0, 0.f, y,
                   topk_idx, topk_w);
}

/* GptOssMoELayer::incremental_forwarding (gpt_oss_moe_layer.cpp:452-568) with the expert of
 * compute_expert_forward_no_critical (:372-449). logits already hold the router bias.
 * gate_bias, up_bias [E][I]; down_bias [E][H]. The reference accumulates weight * expert output
 * per expert and then adds the experts in ascending order, which for one token is the ascending
 * sum of its pairs, as above. */
void orc_moe_forward_gpt_oss(int kind, int renormalize, int T, int H, int I, int E, int topk, const float *x,
                             const float *logits, const void *const *gate, const void *const *up,
                             const void *const *down, const float *gate_bias, const float *up_bias,
                             const float *down_bias, float alpha, float *y, int32_t *topk_idx,
                             float *topk_w) {
  moe_forward_impl(kind, renormalize, T, H, I, E, topk, x, logits, gate, up, down, gate_bias, up_bias, down_bias,
                   1, alpha, y, topk_idx, topk_w);
}

void orc_moe_forward_q4_K(int T, int H, int I, int E, int topk, const float *x,
                          const float *logits, const void *const *gate,
                          const void *const *up, const void *const *down,
                          float *y, int32_t *topk_idx, float *topk_w) {
  orc_moe_forward(12, 1, T, H, I, E, topk, x, logits, gate, up, down, y, topk_idx, topk_w);
}

/* nntrainer::swiglu(N, X, Y, Z): X = (Y / (1 + exp(-Y))) * Z, fp32 with the float exponential
 * (fallback_internal.cpp:417-423; the AVX2 build evaluates the same expression with a polynomial
 * exponential, avx2_impl.cpp:304-311, within the path's tolerance of this one). */
void orc_swiglu(int64_t n, float *x, const float *y, const float *z) {
  for (int64_t i = 0; i < n; ++i) x[i] = (y[i] / (1.f + expf(-y[i]))) * z[i];
}

/* ------------------------------------------------------------------------- */
/* nntrainer::swiglu as an x86 build of the reference evaluates it             */
/* ------------------------------------------------------------------------- */

/* avx2_approx_exp_e2lookup<8>, nntrainer/tensor/cpu_backend/x86/avx2_impl.cpp:227-294:
 * e^x = 2^(k/8) * 2^f with k = nearest integer of 8x/ln2 (read out of the mantissa of
 * x' + 1.5*2^23), 2^(k/8) from an eight-entry table of bit patterns plus k shifted into
 * the exponent, and 2^f - 1 by a cubic in the remainder. One lane of the vector code,
 * operation by operation; the table is the one a C++17 build carries (:166-174). */
static inline float approx_exp_x86(float x) {
  static const uint32_t tbl[8] = {0x3f800000u, 0x3f7b95c2u, 0x3f7837f0u, 0x3f75fed7u,
                                  0x3f7504f3u, 0x3f75672au, 0x3f7744fdu, 0x3f7ac0c7u};
  const float arg_min = -87.0f, arg_max = +88.3762626647949f; /* :142-143 */
  const double ln2 = 0.69314718055994530942; /* M_LN2, what numbers::ln2_v<double> is in a C++17 build (:132-137) */
  const float to_k = (float)(1.0 / ln2 * 8);
  const float k_max = (float)(arg_max / ln2 * 8);
  const float c0 = 0x1.c6af84b912394p-5f / 8 / 8 / 8, c1 = 0x1.ebfce50fac4f3p-3f / 8 / 8,
              c2 = 0x1.62e42ff0c52d6p-1f / 8;
  x = x > arg_min ? x : arg_min; /* _mm256_max_ps(xs, MIN) */
  x = x * to_k;
  x = x < k_max ? x : k_max;     /* _mm256_min_ps(xs, MAX) */
  float xi = x + 0x1.8p23f;
  const uint32_t bits = f32_bits(xi);
  xi = xi - 0x1.8p23f;
  const float fr = x - xi;
  const float sc = bits_f32(tbl[bits & 7u] + (bits << 20));
  const float q0 = fmaf(fr, c0, c1);
  const float fr2 = fr * fr;
  const float q2 = fr * c2;
  const float pl = fmaf(q0, fr2, q2);
  return fmaf(pl, sc, sc);
}

/* avx2::swiglu, avx2_impl.cpp:297-304 and 906-947: X = (Y / (exp'(-Y) + 1)) * Z with the
 * exponential above, denormals read and written as zero while it runs (:909-910). Every
 * lane of the 16-wide, 8-wide and masked steps does the same arithmetic. */
void orc_swiglu_x86(int64_t n, float *x, const float *y, const float *z) {
  const unsigned csr = _mm_getcsr();
  _mm_setcsr(csr | 0x8040u);
  for (int64_t i = 0; i < n; ++i) {
    const float inv = approx_exp_x86(-y[i]) + 1.0f;
    x[i] = (y[i] / inv) * z[i];
  }
  _mm_setcsr(csr);
}

/* avx2::swiglu with alpha, avx2_impl.cpp:306-316 and 950-993: the exponent is -(alpha * Y). */
void orc_swiglu_alpha_x86(int64_t n, float *x, const float *y, const float *z, float alpha) {
  const unsigned csr = _mm_getcsr();
  _mm_setcsr(csr | 0x8040u);
  for (int64_t i = 0; i < n; ++i) {
    const float ay = alpha * y[i];
    const float inv = approx_exp_x86(-ay) + 1.0f;
    x[i] = (y[i] / inv) * z[i];
  }
  _mm_setcsr(csr);
}

/* ------------------------------------------------------------------------- */
/* the cached mixture-of-experts layers                                       */
/* ------------------------------------------------------------------------- */

static void gemm_kind(int kind, int M, int N, int K, const float *A, const void *W, float *C) {
  if (kind == 2)
    orc_gemm_q4_0(M, N, K, A, W, C);
  else if (kind == 12)
    orc_gemm_q4_K(M, N, K, A, W, C);
  else
    orc_gemm_q6_K(M, N, K, A, W, C);
}

/* CachedSlimMoELayer::incremental_forwarding with compute_expert_forward
 * (Applications/CausalLM/layers/qwen_moe_layer_cached.cpp:266-470, 176-265) and, with
 * gpt_oss = 1, CachedSlimGptOssMoELayer (gpt_oss_moe_layer_cached.cpp:193-426, 438-530).
 * Routing as in the plain layers (softmax, top-k, renormalised). Then per expert, in
 * ascending id, ONE product with M = the number of its tokens (their rows gathered in
 * ascending token order; one token: its row where it lies): so rows [0, 4*(M/4)) take
 * the 4-row quantizer and the GEMM kernel's fp32 order and the others the row forms,
 * as in every M > 1 product of the path.
 *   Qwen: one token h = (sigmoid(g) * g) * u with the double-precision sigmoid of the
 *         activation function (:236-241); more tokens nntrainer::swiglu, the x86 form
 *         above (:242-250).
 *   GPT-OSS: g += gate_bias, g = min(g, limit); u += up_bias, u = clamp(u, -limit, limit);
 *         u += 1; nntrainer::swiglu with alpha for every token count; the down product
 *         takes down_bias (:497-530).
 * The expert's weighted rows go into its own zero-filled [T x H] tensor (0 + w * o) and
 * the experts' tensors are added in ascending order (:456-464). */
void orc_moe_forward_cached(int kind, int gpt_oss, int T, int H, int I, int E, int topk, const float *x,
                            const float *logits, const void *const *gate, const void *const *up,
                            const void *const *down, const float *gate_bias, const float *up_bias,
                            const float *down_bias, float alpha, float limit, float *y, int32_t *topk_idx,
                            float *topk_w) {
  int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)T * topk);
  float *wt = (float *)malloc(sizeof(float) * (size_t)T * topk);
  moe_route(1, T, E, topk, logits, idx, wt);
  if (topk_idx) memcpy(topk_idx, idx, sizeof(int32_t) * (size_t)T * topk);
  if (topk_w) memcpy(topk_w, wt, sizeof(float) * (size_t)T * topk);

  int *tok = (int *)malloc(sizeof(int) * (size_t)T);
  float *tw = (float *)malloc(sizeof(float) * (size_t)T);
  float *tin = (float *)malloc(sizeof(float) * (size_t)T * H);
  float *g = (float *)malloc(sizeof(float) * (size_t)T * I);
  float *u = (float *)malloc(sizeof(float) * (size_t)T * I);
  float *h = (float *)malloc(sizeof(float) * (size_t)T * I);
  float *o = (float *)malloc(sizeof(float) * (size_t)T * H);
  float *eo = (float *)malloc(sizeof(float) * (size_t)T * H);
  int first = 1;
  for (int e = 0; e < E; ++e) {
    int n = 0;
    for (int t = 0; t < T; ++t)
      for (int k = 0; k < topk; ++k)
        if (idx[t * topk + k] == e) {
          tok[n] = t;
          tw[n] = wt[t * topk + k];
          ++n;
        }
    if (!n) continue;
    for (int i = 0; i < n; ++i) memcpy(tin + (size_t)i * H, x + (size_t)tok[i] * H, sizeof(float) * (size_t)H);
    gemm_kind(kind, n, I, H, tin, gate[e], g);
    gemm_kind(kind, n, I, H, tin, up[e], u);
    if (gpt_oss) {
      for (int i = 0; i < n; ++i)
        for (int c = 0; c < I; ++c) {
          float gv = g[(size_t)i * I + c] + gate_bias[(size_t)e * I + c];
          gv = gv < limit ? gv : limit; /* clamp(lowest, limit): max with lowest changes nothing */
          float uv = u[(size_t)i * I + c] + up_bias[(size_t)e * I + c];
          uv = uv > -limit ? uv : -limit;
          uv = uv < limit ? uv : limit;
          g[(size_t)i * I + c] = gv;
          u[(size_t)i * I + c] = uv + 1.f;
        }
      for (int i = 0; i < n; ++i)
        orc_swiglu_alpha_x86(I, h + (size_t)i * I, g + (size_t)i * I, u + (size_t)i * I, alpha);
    } else if (n == 1) {
      for (int c = 0; c < I; ++c) {
        const float en = (float)exp((double)(-g[c]));
        const float sig = (float)(1.0 / (1.0 + (double)en));
        h[c] = (sig * g[c]) * u[c];
      }
    } else {
      for (int i = 0; i < n; ++i) orc_swiglu_x86(I, h + (size_t)i * I, g + (size_t)i * I, u + (size_t)i * I);
    }
    gemm_kind(kind, n, H, I, h, down[e], o);
    memset(eo, 0, sizeof(float) * (size_t)T * H);
    for (int i = 0; i < n; ++i)
      for (int c = 0; c < H; ++c) {
        float v = o[(size_t)i * H + c];
        if (gpt_oss) v = v + down_bias[(size_t)e * H + c];
        v = v * tw[i];
        eo[(size_t)tok[i] * H + c] = eo[(size_t)tok[i] * H + c] + v;
      }
    if (first) {
      memcpy(y, eo, sizeof(float) * (size_t)T * H);
      first = 0;
    } else
      for (size_t j = 0; j < (size_t)T * H; ++j) y[j] = y[j] + eo[j];
  }
  if (first) memset(y, 0, sizeof(float) * (size_t)T * H);
  free(tok); free(tw); free(tin); free(g); free(u); free(h); free(o); free(eo); free(idx); free(wt);
}

void orc_set_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}
