// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemv_device.h
 * @brief  Device-side block-dot GEMV engine for Q4_0 x Q8_0, Q4_K x Q8_K and
 *         Q6_K x Q8_K, shared by the decode GEMV kernels and the grouped
 *         mixture-of-experts kernels.
 *
 * Results are bit-identical to the reference's x86 AVX2 kernels
 * (IMPL = nntrainer/tensor/cpu_backend/ggml_interface/nntr_ggml_impl in the
 * reference checkout): integer inner sums are exact, and the fp32 operations
 * per output are the reference's, in the reference's order:
 *   Q4_0: acc = fma(float(isum_b), dw_b * da_b, acc), blocks b ascending
 *         (IMPL/nntr_ggml_impl.cpp:9676-9752, 2878-2901);
 *   Q4_K: acc = fma(float(I), d * dA, acc), accm = fma(float(Im), dmin * dA, accm)
 *         once per super-block (GEMV kernel, :7133-7422) or once per pair of
 *         sub-blocks (GEMM kernel, :6274-6989, used by the reference for rows
 *         [0, 4*(M/4)) when M > 1); result acc - accm;
 *   Q6_K: eight partial accumulators, partial l owning the elements whose index
 *         mod 32 lies in [4l, 4l+4): acc_l = fma(dA * dw, float(S_l), acc_l) per
 *         super-block, then ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)) (:8602-8695).
 *
 * Two phases per wavefront and K-chunk of 4096 weights:
 *   phase 1  T lanes (16 or 64) stream one weight row with 128-bit non-temporal
 *            loads, unpack nibbles in registers and form exact integer partial
 *            sums with v_dot4_i32_i8 against R rows of quantized activations;
 *            partials of a block / sub-block pair are combined over DPP
 *            (integers, exact) and written to LDS as per-block records;
 *   phase 2  one lane per (weight row, activation row) [x 8 for Q6_K] walks the
 *            records of its output in ascending K order and performs the fp32
 *            chain above. G weight rows share one pass so that the sequential
 *            chains run on many lanes at once.
 */
#ifndef HIPQ_GEMV_DEVICE_H
#define HIPQ_GEMV_DEVICE_H

#include "hipq_internal.h"

#define HIPQ_M4 0x0F0F0F0Fu
#define HIPQ_KCHUNK 4096 /* weights per phase-1/phase-2 round */

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

/* Dwords of LDS per (weight row, activation row) and K-chunk. The odd-ish
 * strides keep the phase-2 lanes, which read the same record index of
 * different outputs, on different banks. */
template <int DT> struct GemvRec;
template <> struct GemvRec<HIPQ_Q4_0> {
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 32) * 2 + 2; /* {float isum, float scale} per block */
  static constexpr int LANES_PER_OUT = 1;
};
template <> struct GemvRec<HIPQ_Q4_K> {
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 256) * 10 + 2; /* {I[4], Im[4], sd, sm} per super-block */
  static constexpr int LANES_PER_OUT = 1;
};
template <> struct GemvRec<HIPQ_Q6_K> {
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 256) * 9 + 1; /* {S[8], d} per super-block */
  static constexpr int LANES_PER_OUT = 8;
};

/* ---- phase 1 ---------------------------------------------------------------- */

/* Q4_0: a unit is one 32-value block; a lane owns whole blocks, no cross-lane
 * step is needed. rec points at this weight row's records [R][PER_CHUNK]. */
template <int T, int R>
__device__ __forceinline__ void gemv_p1_q4_0(const WView &w, int row, int tl, const QView &qa,
                                             const int (&arow)[R], int k0, int kc, uint32_t *rec) {
  const int units = w.K >> 5, u0 = k0 >> 5, un = kc >> 5;
  const uint4 *qs = (const uint4 *)w.qs + (size_t)row * units + u0;
  const uint16_t *dw = w.d + (size_t)row * units + u0;
#pragma unroll 2
  for (int u = tl; u < un; u += T) {
    const uint4 q = hipq_ld_stream(qs + u);
    const float d = hipq_h2f(dw[u]);
    const uint32_t lo[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
    const uint32_t hi[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                            (q.w >> 4) & HIPQ_M4};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int4 *a = (const int4 *)(qa.q + (size_t)arow[r] * qa.K + (size_t)(u0 + u) * 32);
      const int4 a0 = a[0], a1 = a[1];
      const uint32_t meta = qa.meta[(size_t)arow[r] * units + u0 + u];
      const float da = hipq_h2f((uint16_t)(meta & 0xffff));
      const int bsum = (int)(int16_t)(meta >> 16);
      const int isum = hipq_dot16(lo, a0) + hipq_dot16(hi, a1) - 8 * bsum; /* weights are nibble - 8 */
      float2 v;
      v.x = (float)isum;
      v.y = d * da;
      *(float2 *)(rec + r * GemvRec<HIPQ_Q4_0>::PER_CHUNK + 2 * u) = v;
    }
  }
}

/* Q4_K: a unit is 16 bytes = halves (h) of sub-blocks 2c and 2c+1 of a
 * super-block; lanes u and u^1 hold the two halves of pair c. */
template <int T, int R>
__device__ __forceinline__ void gemv_p1_q4_K(const WView &w, int row, int tl, const QView &qa,
                                             const int (&arow)[R], int k0, int kc, uint32_t *rec) {
  const int units = w.K >> 5, nsb = w.K >> 8, u0 = k0 >> 5, un = kc >> 5, b0 = k0 >> 8;
  const uint4 *qs = (const uint4 *)w.qs + (size_t)row * units + u0;
  const uint4 *hdr = (const uint4 *)w.hdr + (size_t)row * nsb + b0;
  /* all lanes run the same trip count: the DPP exchange needs both partners */
  const int trips = (un + T - 1) / T;
#pragma unroll 2
  for (int it = 0; it < trips; ++it) {
    const int u = tl + it * T;
    const bool on = u < un;
    const int uc = on ? u : un - 1;
    const int b = uc >> 3, c = (uc >> 1) & 3, h = uc & 1;
    const uint4 q = hipq_ld_stream(qs + uc);
    const uint4 hd = hdr[b];
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
    const int j = 2 * c + h;
    const float dw = hipq_h2f((uint16_t)(hd.x & 0xffff));
    const float dmin = hipq_h2f((uint16_t)(hd.x >> 16));
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int8_t *ab = qa.q + (size_t)arow[r] * qa.K + (size_t)(b0 + b) * 256 + c * 64 + h * 16;
      const int4 alo = *(const int4 *)(ab);
      const int4 ahi = *(const int4 *)(ab + 32);
      int I = sc0 * hipq_dot16(lo, alo) + sc1 * hipq_dot16(hi, ahi);
      const int bsw =
        *(const int *)(qa.bsum + (size_t)arow[r] * (qa.K >> 4) + (b0 + b) * 16 + 2 * j);
      int Im = mn * ((int)(int16_t)(bsw & 0xffff) + (bsw >> 16));
      I += hipq_dpp_i<HIPQ_DPP_XOR1>(I); /* both halves of the sub-block pair */
      Im += hipq_dpp_i<HIPQ_DPP_XOR1>(Im);
      if (on && h == 0) {
        uint32_t *o = rec + r * GemvRec<HIPQ_Q4_K>::PER_CHUNK + b * 10;
        o[c] = (uint32_t)I;
        o[4 + c] = (uint32_t)Im;
        if (c == 0) {
          const float dA = qa.d[(size_t)arow[r] * nsb + b0 + b];
          o[8] = __float_as_uint(dw * dA);
          o[9] = __float_as_uint(dmin * dA);
        }
      }
    }
  }
}

/* Q6_K: a unit is 64 weights = 2 x 16 B of ql + 16 B of qh, unit uu = half*2 + hl
 * of a super-block. Dword t of the unit belongs to partial l = hl*4 + t; lanes
 * uu and uu^2 hold the two halves. */
template <int T, int R>
__device__ __forceinline__ void gemv_p1_q6_K(const WView &w, int row, int tl, const QView &qa,
                                             const int (&arow)[R], int k0, int kc, uint32_t *rec) {
  const int nsb = w.K >> 8, b0 = k0 >> 8, un = kc >> 6;
  const uint8_t *qlrow = w.qs + (size_t)row * (w.K >> 1) + (size_t)b0 * 128;
  const uint8_t *qhrow = w.qh + (size_t)row * (w.K >> 2) + (size_t)b0 * 64;
  const int8_t *scrow = w.sc + (size_t)row * (w.K >> 4) + (size_t)b0 * 16;
  const uint16_t *drow = w.d + (size_t)row * nsb + b0;
  const int trips = (un + T - 1) / T;
  for (int it = 0; it < trips; ++it) {
    const int u = tl + it * T;
    const bool on = u < un;
    const int uc = on ? u : un - 1;
    const int b = uc >> 2, uu = uc & 3, half = uu >> 1, hl = uu & 1;
    const uint8_t *ql = qlrow + b * 128 + half * 64 + hl * 16;
    const uint4 qa_ = hipq_ld_stream((const uint4 *)ql);
    const uint4 qb_ = hipq_ld_stream((const uint4 *)(ql + 32));
    const uint4 qh_ = hipq_ld_stream((const uint4 *)(qhrow + b * 64 + half * 32 + hl * 16));
    const int scw = *(const int *)(scrow + b * 16 + uu * 4);
    const uint32_t A[4] = {qa_.x, qa_.y, qa_.z, qa_.w};
    const uint32_t B[4] = {qb_.x, qb_.y, qb_.z, qb_.w};
    const uint32_t H[4] = {qh_.x, qh_.y, qh_.z, qh_.w};
    const int s0 = (int)(int8_t)(scw & 0xff), s1 = (int)(int8_t)((scw >> 8) & 0xff);
    const int s2 = (int)(int8_t)((scw >> 16) & 0xff), s3 = (int)(int8_t)((scw >> 24) & 0xff);
    const float dwt = hipq_h2f(drow[b]);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int8_t *ab =
        qa.q + (size_t)arow[r] * qa.K + (size_t)(b0 + b) * 256 + half * 128 + hl * 16;
      const int4 a0 = *(const int4 *)(ab), a1 = *(const int4 *)(ab + 32);
      const int4 a2 = *(const int4 *)(ab + 64), a3 = *(const int4 *)(ab + 96);
      const int a0w[4] = {a0.x, a0.y, a0.z, a0.w}, a1w[4] = {a1.x, a1.y, a1.z, a1.w};
      const int a2w[4] = {a2.x, a2.y, a2.z, a2.w}, a3w[4] = {a3.x, a3.y, a3.z, a3.w};
      int P[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        /* 6-bit values of the four 32-element groups, 4 at a time; (q6 - 32) . a
         * = q6 . a - 32 . a, both via v_dot4 */
        const int v0 = (int)((A[t] & HIPQ_M4) | ((H[t] << 4) & 0x30303030u));
        const int v1 = (int)((B[t] & HIPQ_M4) | ((H[t] << 2) & 0x30303030u));
        const int v2 = (int)(((A[t] >> 4) & HIPQ_M4) | (H[t] & 0x30303030u));
        const int v3 = (int)(((B[t] >> 4) & HIPQ_M4) | ((H[t] >> 2) & 0x30303030u));
        const int c32 = 0x20202020;
        int p = s0 * (hipq_dot4(v0, a0w[t], 0) - hipq_dot4(c32, a0w[t], 0));
        p += s1 * (hipq_dot4(v1, a1w[t], 0) - hipq_dot4(c32, a1w[t], 0));
        p += s2 * (hipq_dot4(v2, a2w[t], 0) - hipq_dot4(c32, a2w[t], 0));
        p += s3 * (hipq_dot4(v3, a3w[t], 0) - hipq_dot4(c32, a3w[t], 0));
        P[t] = p + hipq_dpp_i<HIPQ_DPP_XOR2>(p); /* both 128-element halves */
      }
      if (on && half == 0) {
        uint32_t *o = rec + r * GemvRec<HIPQ_Q6_K>::PER_CHUNK + b * 9;
#pragma unroll
        for (int t = 0; t < 4; ++t) o[hl * 4 + t] = (uint32_t)P[t];
        if (hl == 0) o[8] = __float_as_uint(qa.d[(size_t)arow[r] * nsb + b0 + b] * dwt);
      }
    }
  }
}

/* ---- engine ------------------------------------------------------------------ */

struct GemvOut {
  float v;    /* finished output                                   */
  int g, r;   /* weight row within the group, activation row index */
  bool valid; /* this lane carries an output                       */
};

/**
 * Computes, for the G weight rows starting at row0 (clamped to the matrix) and
 * the R activation rows arow[], all G*R outputs. Must be called by every lane
 * of every wavefront of the workgroup (it uses __syncthreads); `lds` is this
 * wavefront's private region of G*R*PER_CHUNK dwords. `pair_rows`: activation
 * rows with arow[r] < pair_rows use the per-sub-block-pair order (Q4_K only).
 */
template <int DT, int T, int R, int G>
__device__ __forceinline__ GemvOut gemv_engine(const WView &w, int row0, const QView &qa,
                                               const int (&arow)[R], int pair_rows,
                                               uint32_t *lds) {
  constexpr int RW = 64 / T; /* weight rows streamed at once */
  constexpr int PER = GemvRec<DT>::PER_CHUNK;
  constexpr int LPO = GemvRec<DT>::LANES_PER_OUT;
  static_assert(G % RW == 0, "group must be a multiple of the rows streamed at once");
  static_assert(G * R * LPO <= 64, "one lane per fp32 chain");
  const int lane = threadIdx.x & 63, tl = lane % T;
  const int ci = lane / LPO, l = lane % LPO; /* chain of this lane in phase 2 */
  const bool chain = ci < G * R;
  const int cg = chain ? ci / R : 0, cr = chain ? ci % R : 0;
  const uint32_t *crec = lds + (cg * R + cr) * PER;
  float acc = 0.f, accm = 0.f;
  const bool pairwise = DT == HIPQ_Q4_K && arow[cr] < pair_rows;

  for (int k0 = 0; k0 < w.K; k0 += HIPQ_KCHUNK) {
    const int kc = min(HIPQ_KCHUNK, w.K - k0);
#pragma unroll
    for (int pass = 0; pass < G / RW; ++pass) {
      const int g = pass * RW + lane / T;
      const int row = min(row0 + g, w.N - 1);
      uint32_t *rec = lds + g * R * PER;
      if (DT == HIPQ_Q4_0)
        gemv_p1_q4_0<T, R>(w, row, tl, qa, arow, k0, kc, rec);
      else if (DT == HIPQ_Q4_K)
        gemv_p1_q4_K<T, R>(w, row, tl, qa, arow, k0, kc, rec);
      else
        gemv_p1_q6_K<T, R>(w, row, tl, qa, arow, k0, kc, rec);
    }
    __syncthreads();
    if (chain) {
      if (DT == HIPQ_Q4_0) {
        const int nb = kc >> 5;
        for (int b = 0; b < nb; ++b) {
          const float2 v = *(const float2 *)(crec + 2 * b);
          acc = fmaf(v.x, v.y, acc);
        }
      } else if (DT == HIPQ_Q4_K) {
        const int nb = kc >> 8;
        for (int b = 0; b < nb; ++b) {
          const uint32_t *o = crec + b * 10;
          const int I0 = (int)o[0], I1 = (int)o[1], I2 = (int)o[2], I3 = (int)o[3];
          const int M0 = (int)o[4], M1 = (int)o[5], M2 = (int)o[6], M3 = (int)o[7];
          const float sd = __uint_as_float(o[8]), sm = __uint_as_float(o[9]);
          if (pairwise) {
            acc = fmaf((float)I0, sd, acc);
            accm = fmaf((float)M0, sm, accm);
            acc = fmaf((float)I1, sd, acc);
            accm = fmaf((float)M1, sm, accm);
            acc = fmaf((float)I2, sd, acc);
            accm = fmaf((float)M2, sm, accm);
            acc = fmaf((float)I3, sd, acc);
            accm = fmaf((float)M3, sm, accm);
          } else {
            acc = fmaf((float)(I0 + I1 + I2 + I3), sd, acc);
            accm = fmaf((float)(M0 + M1 + M2 + M3), sm, accm);
          }
        }
      } else {
        const int nb = kc >> 8;
        for (int b = 0; b < nb; ++b) {
          const uint32_t *o = crec + b * 9;
          acc = fmaf(__uint_as_float(o[8]), (float)(int)o[l], acc);
        }
      }
    }
    __syncthreads();
  }

  GemvOut out;
  out.g = cg;
  out.r = cr;
  if (DT == HIPQ_Q4_K) {
    out.v = acc - accm;
    out.valid = chain;
  } else if (DT == HIPQ_Q6_K) {
    /* ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)) */
    float v = acc;
    v = v + __shfl_xor(v, 4, 64);
    v = v + __shfl_xor(v, 2, 64);
    v = v + __shfl_xor(v, 1, 64);
    out.v = v;
    out.valid = chain && l == 0;
  } else {
    out.v = acc;
    out.valid = chain;
  }
  return out;
}

/* Weight rows per group for a given number of activation rows: G * R fp32
 * chains per wavefront (16 for Q4_K, whose records are small; 8 otherwise),
 * at most 8 rows. */
template <int DT, int R> struct GemvGroup {
  static constexpr int CHAINS = DT == HIPQ_Q4_K ? 16 : 8;
  static constexpr int G = (CHAINS / R) >= 8 ? 8 : (CHAINS / R);
  static constexpr int LDS_DWORDS = G * R * GemvRec<DT>::PER_CHUNK; /* per wavefront */
  /* 16 lanes per weight row stream 4 rows at once, so G must be a multiple of 4 */
  static constexpr bool T16_OK = (G % 4) == 0;
};

#endif /* HIPQ_GEMV_DEVICE_H */
