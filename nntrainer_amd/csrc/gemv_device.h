// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemv_device.h
 * @brief  Device-side block-dot GEMV bodies for Q4_0 x Q8_0, Q4_K x Q8_K and
 *         Q6_K x Q8_K, shared by the decode GEMV kernels and the grouped
 *         mixture-of-experts kernels.
 *
 * A group of T lanes (T = 16 or 64) owns one weight row (one output column).
 * Each lane streams 16-byte units of packed weights with 128-bit non-temporal
 * loads, unpacks nibbles in registers, multiplies against R rows of quantized
 * activations with v_dot4_i32_i8 (exact int32), applies the block scales in
 * fp32 and the group is reduced over DPP. The arithmetic per output is the
 * reference's (IMPL = nntrainer/tensor/cpu_backend/ggml_interface/nntr_ggml_impl
 * in the reference checkout):
 *   Q4_0: sum_b float(isum_b) * (dw_b * da_b)              IMPL/nntr_ggml_impl.cpp:9676-9752
 *   Q4_K: sum_b float(I_b) * (d_b * dA_b)
 *         - sum_b float(Im_b) * (dmin_b * dA_b)            IMPL/nntr_ggml_impl.cpp:7133-7422
 *   Q6_K: sum_b (dA_b * dw_b) * float(S_b)                 IMPL/nntr_ggml_impl.cpp:8602-8695
 * with exact integer inner sums; only the order of the fp32 additions differs
 * (per-lane partial sums, then a fixed reduction tree).
 */
#ifndef HIPQ_GEMV_DEVICE_H
#define HIPQ_GEMV_DEVICE_H

#include "hipq_internal.h"

#define HIPQ_M4 0x0F0F0F0Fu

/* Read-only view of quantized activations for device code. */
struct QView {
  const int8_t *q;
  const uint32_t *meta;
  const float *d;
  const int16_t *bsum;
  int K;
};
static inline QView qview(const QAct &a) {
  QView v;
  v.q = a.q;
  v.meta = a.meta;
  v.d = a.d;
  v.bsum = a.bsum;
  v.K = a.K;
  return v;
}

__device__ __forceinline__ int hipq_dot16(const uint32_t (&w)[4], const int4 &a) {
  int s = hipq_dot4((int)w[0], a.x, 0);
  s = hipq_dot4((int)w[1], a.y, s);
  s = hipq_dot4((int)w[2], a.z, s);
  s = hipq_dot4((int)w[3], a.w, s);
  return s;
}

/* ---- Q4_0 ----------------------------------------------------------------- */
template <int T, int R>
__device__ __forceinline__ void gemv_q4_0_rows(const WView &w, int row, int tl,
                                               const QView &qa, const int (&arow)[R],
                                               float (&out)[R]) {
  const int units = w.K >> 5;
  const uint4 *qs = (const uint4 *)w.qs + (size_t)row * units;
  const uint16_t *dw = w.d + (size_t)row * units;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
#pragma unroll 2
  for (int u = tl; u < units; u += T) {
    const uint4 q = hipq_ld_stream(qs + u);
    const float d = hipq_h2f(dw[u]);
    const uint32_t lo[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
    const uint32_t hi[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                            (q.w >> 4) & HIPQ_M4};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int4 *a = (const int4 *)(qa.q + (size_t)arow[r] * qa.K + (size_t)u * 32);
      const int4 a0 = a[0], a1 = a[1];
      const uint32_t meta = qa.meta[(size_t)arow[r] * units + u];
      const float da = hipq_h2f((uint16_t)(meta & 0xffff));
      const int bsum = (int)(int16_t)(meta >> 16);
      int isum = hipq_dot16(lo, a0) + hipq_dot16(hi, a1);
      isum -= 8 * bsum; /* weights are nibble - 8 */
      acc[r] = fmaf((float)isum, d * da, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = hipq_group_sum<T>(acc[r]);
}

/* ---- Q4_K ----------------------------------------------------------------- */
template <int T, int R>
__device__ __forceinline__ void gemv_q4_K_rows(const WView &w, int row, int tl,
                                               const QView &qa, const int (&arow)[R],
                                               float (&out)[R]) {
  const int units = w.K >> 5; /* 16 bytes = 32 nibbles each */
  const int nsb = w.K >> 8;
  const uint4 *qs = (const uint4 *)w.qs + (size_t)row * units;
  const uint4 *hdr = (const uint4 *)w.hdr + (size_t)row * nsb;
  float acc[R], accm[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = accm[r] = 0.f;
#pragma unroll 2
  for (int u = tl; u < units; u += T) {
    const int b = u >> 3, c = (u >> 1) & 3, h = u & 1;
    const uint4 q = hipq_ld_stream(qs + u);
    const uint4 hd = hdr[b];
    const float d = hipq_h2f((uint16_t)(hd.x & 0xffff));
    const float dmin = hipq_h2f((uint16_t)(hd.x >> 16));
    /* 6-bit scales / mins of sub-blocks 2c and 2c+1 (two adjacent bytes) */
    uint32_t scw, mnw;
    if (c < 2) {
      scw = (hd.y >> (16 * c)) & 0x3f3fu;
      mnw = (hd.z >> (16 * c)) & 0x3f3fu;
    } else {
      const int sh = 16 * (c - 2);
      scw = ((hd.w >> sh) & 0x0f0fu) | ((((hd.y >> sh) >> 6) & 0x0303u) << 4);
      mnw = (((hd.w >> sh) >> 4) & 0x0f0fu) | ((((hd.z >> sh) >> 6) & 0x0303u) << 4);
    }
    const int sc0 = (int)(scw & 0xff), sc1 = (int)(scw >> 8);
    const int mn = (int)((mnw >> (8 * h)) & 0xff);
    const uint32_t lo[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
    const uint32_t hi[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                            (q.w >> 4) & HIPQ_M4};
    const int j = 2 * c + h; /* sub-block whose min term this lane adds */
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int8_t *ab = qa.q + (size_t)arow[r] * qa.K + (size_t)b * 256 + c * 64 + h * 16;
      const int4 alo = *(const int4 *)(ab);
      const int4 ahi = *(const int4 *)(ab + 32);
      const int I = sc0 * hipq_dot16(lo, alo) + sc1 * hipq_dot16(hi, ahi);
      const int bsw = *(const int *)(qa.bsum + (size_t)arow[r] * (qa.K >> 4) + b * 16 + 2 * j);
      const int bs = (int)(int16_t)(bsw & 0xffff) + (bsw >> 16);
      const float dA = qa.d[(size_t)arow[r] * nsb + b];
      acc[r] = fmaf((float)I, d * dA, acc[r]);
      accm[r] = fmaf((float)(mn * bs), dmin * dA, accm[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = hipq_group_sum<T>(acc[r]) - hipq_group_sum<T>(accm[r]);
}

/* ---- Q6_K ----------------------------------------------------------------- */
template <int T, int R>
__device__ __forceinline__ void gemv_q6_K_rows(const WView &w, int row, int tl,
                                               const QView &qa, const int (&arow)[R],
                                               float (&out)[R]) {
  const int units = w.K >> 6; /* 64 weights: 2 x 16 B of ql + 16 B of qh */
  const int nsb = w.K >> 8;
  const uint8_t *qlrow = w.qs + (size_t)row * (w.K >> 1);
  const uint8_t *qhrow = w.qh + (size_t)row * (w.K >> 2);
  const int8_t *scrow = w.sc + (size_t)row * (w.K >> 4);
  const uint16_t *drow = w.d + (size_t)row * nsb;
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  for (int u = tl; u < units; u += T) {
    const int b = u >> 2, uu = u & 3, half = uu >> 1, hl = uu & 1;
    const uint8_t *ql = qlrow + b * 128 + half * 64 + hl * 16;
    const uint4 qa_ = hipq_ld_stream((const uint4 *)ql);
    const uint4 qb_ = hipq_ld_stream((const uint4 *)(ql + 32));
    const uint4 qh_ = hipq_ld_stream((const uint4 *)(qhrow + b * 64 + half * 32 + hl * 16));
    const int scw = *(const int *)(scrow + b * 16 + uu * 4);
    const float d = hipq_h2f(drow[b]);
    const uint32_t A[4] = {qa_.x, qa_.y, qa_.z, qa_.w};
    const uint32_t B[4] = {qb_.x, qb_.y, qb_.z, qb_.w};
    const uint32_t H[4] = {qh_.x, qh_.y, qh_.z, qh_.w};
    uint32_t v0[4], v1[4], v2[4], v3[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v0[t] = (A[t] & HIPQ_M4) | ((H[t] << 4) & 0x30303030u);
      v1[t] = (B[t] & HIPQ_M4) | ((H[t] << 2) & 0x30303030u);
      v2[t] = ((A[t] >> 4) & HIPQ_M4) | (H[t] & 0x30303030u);
      v3[t] = ((B[t] >> 4) & HIPQ_M4) | ((H[t] >> 2) & 0x30303030u);
    }
    const int s0 = (int)(int8_t)(scw & 0xff), s1 = (int)(int8_t)((scw >> 8) & 0xff);
    const int s2 = (int)(int8_t)((scw >> 16) & 0xff), s3 = (int)(int8_t)((scw >> 24) & 0xff);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int8_t *ab = qa.q + (size_t)arow[r] * qa.K + (size_t)b * 256 + half * 128 + hl * 16;
      const int4 a0 = *(const int4 *)(ab), a1 = *(const int4 *)(ab + 32);
      const int4 a2 = *(const int4 *)(ab + 64), a3 = *(const int4 *)(ab + 96);
      /* sums of 16 activations, groups half*8 + 2g + hl, g = 0..3 */
      const uint4 bw =
        *(const uint4 *)(qa.bsum + (size_t)arow[r] * (qa.K >> 4) + b * 16 + half * 8);
      const int b0 = hl ? ((int)bw.x >> 16) : (int)(int16_t)(bw.x & 0xffff);
      const int b1 = hl ? ((int)bw.y >> 16) : (int)(int16_t)(bw.y & 0xffff);
      const int b2 = hl ? ((int)bw.z >> 16) : (int)(int16_t)(bw.z & 0xffff);
      const int b3 = hl ? ((int)bw.w >> 16) : (int)(int16_t)(bw.w & 0xffff);
      int S = s0 * (hipq_dot16(v0, a0) - 32 * b0);
      S += s1 * (hipq_dot16(v1, a1) - 32 * b1);
      S += s2 * (hipq_dot16(v2, a2) - 32 * b2);
      S += s3 * (hipq_dot16(v3, a3) - 32 * b3);
      const float dA = qa.d[(size_t)arow[r] * nsb + b];
      acc[r] = fmaf(dA * d, (float)S, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = hipq_group_sum<T>(acc[r]);
}

template <int DT, int T, int R>
__device__ __forceinline__ void gemv_rows(const WView &w, int row, int tl, const QView &qa,
                                          const int (&arow)[R], float (&out)[R]) {
  if (DT == HIPQ_Q4_0)
    gemv_q4_0_rows<T, R>(w, row, tl, qa, arow, out);
  else if (DT == HIPQ_Q4_K)
    gemv_q4_K_rows<T, R>(w, row, tl, qa, arow, out);
  else
    gemv_q6_K_rows<T, R>(w, row, tl, qa, arow, out);
}

#endif /* HIPQ_GEMV_DEVICE_H */
