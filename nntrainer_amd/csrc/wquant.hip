// SPDX-License-Identifier: Apache-2.0
/**
 * @file   wquant.hip
 * @brief  Offline weight quantizers fp32 -> Q4_0 / Q4_K / Q6_K blocks on the GPU.
 *
 * GPU form of quantize_q4_0 / quantize_q4_K / quantize_q6_K
 * (nntrainer/tensor/cpu_backend/x86/x86_compute_backend.cpp:343-370 in the
 * reference checkout), i.e. of quantize_row_q4_0_ref, quantize_row_q4_K_ref with
 * make_qkx2_quants and quantize_row_q6_K_ref with make_qx_quants
 * (nntr_ggml_impl/nntr_ggml_impl_quant.cpp:382-418, 901-979 + 115-200,
 * 1116-1186 + 32-113). Not on the inference path: it exists so that model
 * preparation and the benchmark do not need a CPU quantizer. One thread
 * quantizes one block; all arithmetic is scalar fp32 with the same operation
 * order and the same fused multiply-adds as the reference's x86 GCC build, so
 * the emitted bytes are identical to the reference's.
 */
#include "hipq_internal.h"

namespace {

constexpr float kMagic = 12582912.f;

__device__ __forceinline__ int magic_int(float biased) {
  return (int)(__float_as_uint(biased) & 0x007fffffu) - 0x00400000;
}
__device__ __forceinline__ int nearest_plain(float v) { return magic_int(__fadd_rn(v, kMagic)); }
__device__ __forceinline__ int nearest_prod(float a, float b) {
  return magic_int(__fmaf_rn(a, b, kMagic));
}

__global__ void quantize_w_q4_0(const float *__restrict__ src, int64_t nblk,
                                uint8_t *__restrict__ dst) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblk) return;
  const float *x = src + b * 32;
  uint8_t *y = dst + b * 18;
  float amax = 0.f, vmax = 0.f;
  for (int j = 0; j < 32; ++j) {
    const float a = fabsf(x[j]);
    if (amax < a) {
      amax = a;
      vmax = x[j];
    }
  }
  /* max / -8 as an exact scaling plus a sign flip (keeps -0 for an all-zero block) */
  const float d = -(vmax * 0.125f);
  const float id = d != 0.f ? __fdiv_rn(1.0f, d) : 0.0f;
  const uint16_t hd = hipq_f2h(d);
  y[0] = (uint8_t)(hd & 0xff);
  y[1] = (uint8_t)(hd >> 8);
  for (int j = 0; j < 16; ++j) {
    const int lo = min(15, (int)(int8_t)(int)__fmaf_rn(x[j], id, 8.5f));
    const int hi = min(15, (int)(int8_t)(int)__fmaf_rn(x[j + 16], id, 8.5f));
    y[2 + j] = (uint8_t)(lo | (hi << 4));
  }
}

/* scale/min search of one 32-value sub-block (make_qkx2_quants, n=32, nmax=15,
 * rmin=-1, rdelta=0.1, nstep=20, squared error) */
__device__ float q4k_fit(const float *x, const float *w, uint8_t *L, float *neg_min) {
  float lo = x[0], hi = x[0];
  float sum_w = w[0];
  float sum_x = __fmul_rn(sum_w, x[0]);
  for (int i = 1; i < 32; ++i) {
    if (x[i] < lo) lo = x[i];
    if (x[i] > hi) hi = x[i];
    sum_w = __fadd_rn(sum_w, w[i]);
    sum_x = __fmaf_rn(w[i], x[i], sum_x);
  }
  if (lo > 0) lo = 0;
  if (hi == lo) {
    for (int i = 0; i < 32; ++i) L[i] = 0;
    *neg_min = -lo;
    return 0.f;
  }
  float iscale = __fdiv_rn(15.f, __fsub_rn(hi, lo));
  float scale = __fdiv_rn(1.f, iscale);
  float best = 0;
  for (int i = 0; i < 32; ++i) {
    const int l = nearest_prod(iscale, __fsub_rn(x[i], lo));
    L[i] = (uint8_t)max(0, min(15, l));
    float diff = __fsub_rn(__fmaf_rn(scale, (float)L[i], lo), x[i]);
    diff = __fmul_rn(diff, diff);
    best = __fmaf_rn(w[i], diff, best);
  }
  uint8_t Laux[32];
  for (int is = 0; is <= 20; ++is) {
    iscale = __fdiv_rn(__fadd_rn(__fmaf_rn(0.1f, (float)is, -1.f), 15.f), __fsub_rn(hi, lo));
    float sum_l = 0, sum_l2 = 0, sum_xl = 0;
    for (int i = 0; i < 32; ++i) {
      int l = nearest_prod(iscale, __fsub_rn(x[i], lo));
      l = max(0, min(15, l));
      Laux[i] = (uint8_t)l;
      const float wl = __fmul_rn(w[i], (float)l);
      sum_l = __fadd_rn(sum_l, wl);
      sum_l2 = __fmaf_rn(wl, (float)l, sum_l2);
      sum_xl = __fmaf_rn(wl, x[i], sum_xl);
    }
    const float D = __fmaf_rn(sum_w, sum_l2, -__fmul_rn(sum_l, sum_l));
    if (D > 0) {
      float this_scale = __fdiv_rn(__fmaf_rn(-sum_x, sum_l, __fmul_rn(sum_w, sum_xl)), D);
      float this_min = __fdiv_rn(__fmaf_rn(sum_l2, sum_x, -__fmul_rn(sum_l, sum_xl)), D);
      if (this_min > 0) {
        this_min = 0;
        this_scale = __fdiv_rn(sum_xl, sum_l2);
      }
      float err = 0;
      for (int i = 0; i < 32; ++i) {
        float diff = __fsub_rn(__fmaf_rn(this_scale, (float)Laux[i], this_min), x[i]);
        diff = __fmul_rn(diff, diff);
        err = __fmaf_rn(w[i], diff, err);
      }
      if (err < best) {
        for (int i = 0; i < 32; ++i) L[i] = Laux[i];
        best = err;
        scale = this_scale;
        lo = this_min;
      }
    }
  }
  *neg_min = -lo;
  return scale;
}

__device__ __forceinline__ void get_scale_min(int j, const uint8_t *s, int &sc, int &mn) {
  if (j < 4) {
    sc = s[j] & 63;
    mn = s[j + 4] & 63;
  } else {
    sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
    mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
  }
}

__global__ __launch_bounds__(64) void quantize_w_q4_K(const float *__restrict__ src, int64_t nblk,
                                                      uint8_t *__restrict__ dst) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblk) return;
  const float *x = src + b * 256;
  uint8_t *y = dst + b * 144;
  uint8_t L[256];
  float w[32], mins[8], scales[8];
  float max_scale = 0, max_min = 0;
  for (int j = 0; j < 8; ++j) {
    const float *xs = x + 32 * j;
    float sum_x2 = 0;
    for (int l = 0; l < 32; ++l) sum_x2 = __fmaf_rn(xs[l], xs[l], sum_x2);
    /* sqrtf: correctly rounded (the __fsqrt_rn intrinsic maps to the native approximation) */
    const float av_x = sqrtf(__fdiv_rn(sum_x2, 32.f));
    for (int l = 0; l < 32; ++l) w[l] = __fadd_rn(av_x, fabsf(xs[l]));
    scales[j] = q4k_fit(xs, w, L + 32 * j, &mins[j]);
    if (scales[j] > max_scale) max_scale = scales[j];
    if (mins[j] > max_min) max_min = mins[j];
  }
  const float inv_scale = max_scale > 0 ? __fdiv_rn(63.f, max_scale) : 0.f;
  const float inv_min = max_min > 0 ? __fdiv_rn(63.f, max_min) : 0.f;
  uint8_t sc[12];
  for (int k = 0; k < 12; ++k) sc[k] = 0;
  for (int j = 0; j < 8; ++j) {
    int ls = (uint8_t)nearest_prod(inv_scale, scales[j]);
    int lm = (uint8_t)nearest_prod(inv_min, mins[j]);
    ls = min(63, ls);
    lm = min(63, lm);
    if (j < 4) {
      sc[j] = (uint8_t)ls;
      sc[j + 4] = (uint8_t)lm;
    } else {
      sc[j + 4] = (uint8_t)((ls & 0x0f) | ((lm & 0x0f) << 4));
      sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
      sc[j] |= (uint8_t)((lm >> 4) << 6);
    }
  }
  const uint16_t hd = hipq_f2h(__fdiv_rn(max_scale, 63.f));
  const uint16_t hm = hipq_f2h(__fdiv_rn(max_min, 63.f));
  y[0] = (uint8_t)(hd & 0xff);
  y[1] = (uint8_t)(hd >> 8);
  y[2] = (uint8_t)(hm & 0xff);
  y[3] = (uint8_t)(hm >> 8);
  for (int k = 0; k < 12; ++k) y[4 + k] = sc[k];
  const float fd = hipq_h2f(hd), fm = hipq_h2f(hm);
  for (int j = 0; j < 8; ++j) {
    int s, m;
    get_scale_min(j, sc, s, m);
    const float d = __fmul_rn(fd, (float)s);
    if (d == 0.f) continue;
    const float dm = __fmul_rn(fm, (float)m);
    for (int i = 0; i < 32; ++i) {
      const int l = nearest_plain(__fdiv_rn(__fadd_rn(x[32 * j + i], dm), d));
      L[32 * j + i] = (uint8_t)max(0, min(15, l));
    }
  }
  for (int c = 0; c < 4; ++c)
    for (int l = 0; l < 32; ++l)
      y[16 + 32 * c + l] = (uint8_t)(L[64 * c + l] | (L[64 * c + 32 + l] << 4));
}

/* symmetric scale search of one 16-value group (make_qx_quants, n=16, nmax=32,
 * rmse_type=1, weights x^2) */
__device__ float q6k_fit(const float *x, int8_t *L) {
  float vmax = 0, amax = 0;
  for (int i = 0; i < 16; ++i) {
    const float a = fabsf(x[i]);
    if (a > amax) {
      amax = a;
      vmax = x[i];
    }
  }
  if (amax < 1e-15f) {
    for (int i = 0; i < 16; ++i) L[i] = 0;
    return 0.f;
  }
  float iscale = __fdiv_rn(-32.f, vmax);
  float sumlx = 0, suml2 = 0;
  for (int i = 0; i < 16; ++i) {
    int l = nearest_prod(iscale, x[i]);
    l = max(-32, min(31, l));
    L[i] = (int8_t)(l + 32);
    const float w = __fmul_rn(x[i], x[i]);
    sumlx = __fmaf_rn(__fmul_rn(w, x[i]), (float)l, sumlx);
    suml2 = __fmaf_rn(__fmul_rn(w, (float)l), (float)l, suml2);
  }
  float scale = suml2 != 0.f ? __fdiv_rn(sumlx, suml2) : 0.0f;
  float best = __fmul_rn(scale, sumlx);
  for (int is = -9; is <= 9; ++is) {
    if (is == 0) continue;
    iscale = __fdiv_rn(-__fmaf_rn(0.1f, (float)is, 32.f), vmax);
    sumlx = suml2 = 0;
    for (int i = 0; i < 16; ++i) {
      int l = nearest_prod(iscale, x[i]);
      l = max(-32, min(31, l));
      const float w = __fmul_rn(x[i], x[i]);
      sumlx = __fmaf_rn(__fmul_rn(w, x[i]), (float)l, sumlx);
      suml2 = __fmaf_rn(__fmul_rn(w, (float)l), (float)l, suml2);
    }
    if (suml2 > 0 && __fmul_rn(sumlx, sumlx) > __fmul_rn(best, suml2)) {
      for (int i = 0; i < 16; ++i) {
        const int l = nearest_prod(iscale, x[i]);
        L[i] = (int8_t)(32 + max(-32, min(31, l)));
      }
      scale = __fdiv_rn(sumlx, suml2);
      best = __fmul_rn(scale, sumlx);
    }
  }
  return scale;
}

__global__ __launch_bounds__(64) void quantize_w_q6_K(const float *__restrict__ src, int64_t nblk,
                                                      uint8_t *__restrict__ dst) {
  const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblk) return;
  const float *x = src + b * 256;
  uint8_t *y = dst + b * 210;
  int8_t L[256];
  float scales[16];
  float max_scale = 0, max_abs = 0;
  for (int g = 0; g < 16; ++g) {
    scales[g] = q6k_fit(x + 16 * g, L + 16 * g);
    const float a = fabsf(scales[g]);
    if (a > max_abs) {
      max_abs = a;
      max_scale = scales[g];
    }
  }
  if (max_abs < 1e-15f) {
    for (int k = 0; k < 210; ++k) y[k] = 0;
    return;
  }
  const float iscale = __fdiv_rn(-128.f, max_scale);
  const uint16_t hd = hipq_f2h(__fdiv_rn(1.f, iscale));
  y[208] = (uint8_t)(hd & 0xff);
  y[209] = (uint8_t)(hd >> 8);
  int8_t sc[16];
  for (int g = 0; g < 16; ++g) {
    sc[g] = (int8_t)min(127, nearest_prod(iscale, scales[g]));
    y[192 + g] = (uint8_t)sc[g];
  }
  const float fd = hipq_h2f(hd);
  for (int g = 0; g < 16; ++g) {
    const float d = __fmul_rn(fd, (float)sc[g]);
    if (d == 0.f) continue;
    for (int i = 0; i < 16; ++i) {
      int l = nearest_plain(__fdiv_rn(x[16 * g + i], d));
      l = max(-32, min(31, l));
      L[16 * g + i] = (int8_t)(l + 32);
    }
  }
  for (int half = 0; half < 2; ++half) {
    const int8_t *Lh = L + 128 * half;
    for (int l = 0; l < 32; ++l) {
      const int q1 = Lh[l] & 0xf, q2 = Lh[l + 32] & 0xf;
      const int q3 = Lh[l + 64] & 0xf, q4 = Lh[l + 96] & 0xf;
      y[64 * half + l] = (uint8_t)(q1 | (q3 << 4));
      y[64 * half + 32 + l] = (uint8_t)(q2 | (q4 << 4));
      y[128 + 32 * half + l] = (uint8_t)((Lh[l] >> 4) | ((Lh[l + 32] >> 4) << 2) |
                                         ((Lh[l + 64] >> 4) << 4) | ((Lh[l + 96] >> 4) << 6));
    }
  }
}

} // namespace

namespace hipq {

int launch_quantize_weights(int dtype, const float *W, int64_t N, int64_t K, void *out,
                            hipStream_t s) {
  if (dtype == HIPQ_Q4_0) {
    const int64_t nblk = N * (K / 32);
    hipq::launch_kernel("quantize_w_q4_0", quantize_w_q4_0, dim3((unsigned)((nblk + 255) / 256)), dim3(256), 0, s, W,
                       nblk, (uint8_t *)out);
  } else if (dtype == HIPQ_Q4_K) {
    const int64_t nblk = N * (K / 256);
    hipq::launch_kernel("quantize_w_q4_K", quantize_w_q4_K, dim3((unsigned)((nblk + 63) / 64)), dim3(64), 0, s, W, nblk,
                       (uint8_t *)out);
  } else if (dtype == HIPQ_Q6_K) {
    const int64_t nblk = N * (K / 256);
    hipq::launch_kernel("quantize_w_q6_K", quantize_w_q6_K, dim3((unsigned)((nblk + 63) / 64)), dim3(64), 0, s, W, nblk,
                       (uint8_t *)out);
  } else {
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", dtype);
  }
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
