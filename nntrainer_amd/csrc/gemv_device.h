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
 *            partials of a block / sub-block pair / super-block are combined
 *            over DPP (integers, exact) and written to LDS as per-block records.
 *            The activations a lane needs are the same for every weight row, so
 *            they are loaded into registers once per chunk; the weight loads of
 *            all rows of the group are issued before the first is consumed.
 *   phase 2  one lane per (weight row, activation row) [x 8 for Q6_K] walks the
 *            records of its output in ascending K order and performs the fp32
 *            chain above. G weight rows share one pass so that the sequential
 *            chains run on several lanes at once.
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
  const uint8_t *ql, *qh; /* Q8_K as 4-bit digits: q = 16 * (qh - 8) + ql */
  int K;
};
static inline QView qview(const QAct &a) {
  QView v;
  v.q = a.q;
  v.meta = a.meta;
  v.d = a.d;
  v.bsum = a.bsum;
  v.ql = a.ql;
  v.qh = a.qh;
  v.K = a.K;
  return v;
}

/* Exact dot product of one Q4_K sub-block (32 unsigned 4-bit weights, eight per
 * dword) with 32 int8 activations given as 4-bit digits lo in 0..15 and
 * hi = (q >> 4) + 8 in 0..15:  sum w*q = 16*sum w*hi + sum w*lo - 128*sum w.
 * Three v_dot8_u32_u4 per eight weights and no nibble unpacking. */
__device__ __forceinline__ int hipq_dot32_u4(const uint4 &w, const uint4 &lo, const uint4 &hi) {
  uint32_t l = __builtin_amdgcn_udot8(w.x, lo.x, 0u, false);
  uint32_t h = __builtin_amdgcn_udot8(w.x, hi.x, 0u, false);
  uint32_t s = __builtin_amdgcn_udot8(w.x, 0x11111111u, 0u, false);
  l = __builtin_amdgcn_udot8(w.y, lo.y, l, false);
  h = __builtin_amdgcn_udot8(w.y, hi.y, h, false);
  s = __builtin_amdgcn_udot8(w.y, 0x11111111u, s, false);
  l = __builtin_amdgcn_udot8(w.z, lo.z, l, false);
  h = __builtin_amdgcn_udot8(w.z, hi.z, h, false);
  s = __builtin_amdgcn_udot8(w.z, 0x11111111u, s, false);
  l = __builtin_amdgcn_udot8(w.w, lo.w, l, false);
  h = __builtin_amdgcn_udot8(w.w, hi.w, h, false);
  s = __builtin_amdgcn_udot8(w.w, 0x11111111u, s, false);
  return (int)((h << 4) + l) - (int)(s << 7);
}

__device__ __forceinline__ int hipq_dot16(const uint32_t (&w)[4], const int4 &a) {
  int s = hipq_dot4((int)w[0], a.x, 0);
  s = hipq_dot4((int)w[1], a.y, s);
  s = hipq_dot4((int)w[2], a.z, s);
  s = hipq_dot4((int)w[3], a.w, s);
  return s;
}

/* ---- per-format traits --------------------------------------------------------- */
/* UNIT: weights covered by one lane-unit. PER_CHUNK: dwords of LDS per (weight
 * row, activation row) and K-chunk; the strides keep the phase-2 lanes, which
 * read the same record index of different outputs, on different banks.
 * PW = records per sub-block pair (needed when some rows use the pairwise order). */
template <int DT, bool PW> struct GemvRec;
template <bool PW> struct GemvRec<HIPQ_Q4_0, PW> {
  static constexpr int UNIT = 32;
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 32) * 2 + 2; /* {float isum, float scale} per block */
  static constexpr int LANES_PER_OUT = 1;
};
template <> struct GemvRec<HIPQ_Q4_K, false> {
  static constexpr int UNIT = 32;
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 256) * 4 + 4; /* {fI, sd, fIm, sm} per super-block */
  static constexpr int LANES_PER_OUT = 1;
};
template <> struct GemvRec<HIPQ_Q4_K, true> {
  static constexpr int UNIT = 32;
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 256) * 10 + 2; /* {I[4], Im[4], sd, sm} per super-block */
  static constexpr int LANES_PER_OUT = 1;
};
template <bool PW> struct GemvRec<HIPQ_Q6_K, PW> {
  static constexpr int UNIT = 64;
  static constexpr int PER_CHUNK = (HIPQ_KCHUNK / 256) * 9 + 1; /* {S[8], d} per super-block */
  static constexpr int LANES_PER_OUT = 8;
};

/* Units a lane handles per chunk of KC weights: 64 lanes cover a 4096-weight chunk
 * in 2 (Q4_0, Q4_K) or 1 (Q6_K) steps. Kernels for short rows (MoE experts) pick
 * fewer lanes per row and a smaller chunk so that no lane and no register idles. */
template <int DT, int T, int KC> struct GemvUnits {
  static constexpr int MAXU = (KC / GemvRec<DT, false>::UNIT + T - 1) / T;
  static_assert(KC <= HIPQ_KCHUNK && KC % 256 == 0, "chunk must fit the LDS records");
};

/* ---- Q4_0 ----------------------------------------------------------------------- */
/* A zero the compiler cannot see through, produced where the call stands: a value
 * combined with it cannot be computed before that point. */
__device__ __forceinline__ uint32_t hipq_late_zero() {
  uint32_t z;
  asm volatile("v_mov_b32 %0, 0" : "=v"(z) : : "memory");
  return z;
}

template <int T, int R, bool PW, int KC> struct GemvQ40 {
  static constexpr int MAXU = GemvUnits<HIPQ_Q4_0, T, KC>::MAXU;
  static constexpr int PER = GemvRec<HIPQ_Q4_0, PW>::PER_CHUNK;
  struct Act {
    int4 a0[MAXU][R], a1[MAXU][R];
    uint32_t meta[MAXU][R]; /* fp16 d | int16 block sum << 16, decoded where it is used: arithmetic on a
                               loaded value here would make the loads behind it wait for it */
  };
  struct Wt {
    uint4 q[MAXU];
    uint32_t d[MAXU]; /* the fp16 scale in a register of its own: two 16-bit loads into the halves of
                         one register would have to wait for each other */
  };
  __device__ static __forceinline__ void load_act(Act &A, const QView &qa, const int (&arow)[R],
                                                  int tl, int k0, int kc) {
    const int units = qa.K >> 5, u0 = k0 >> 5, un = kc >> 5;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break; /* uniform: this step lies beyond the chunk */
      const int u = min(tl + i * T, un - 1);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int4 *a = (const int4 *)(qa.q + (size_t)arow[r] * qa.K + (size_t)(u0 + u) * 32);
        A.a0[i][r] = a[0];
        A.a1[i][r] = a[1];
        A.meta[i][r] = qa.meta[(size_t)arow[r] * units + u0 + u];
      }
    }
  }
  __device__ static __forceinline__ void load_w(Wt &W, const WView &w, int row, int tl, int k0,
                                                int kc) {
    const int units = w.K >> 5, u0 = k0 >> 5, un = kc >> 5;
    const uint4 *qs = (const uint4 *)w.qs + (size_t)row * units + u0;
    const uint16_t *dw = w.d + (size_t)row * units + u0;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = min(tl + i * T, un - 1);
      W.q[i] = hipq_ld_stream(qs + u);
      W.d[i] = hipq_ld_global(dw + u);
    }
  }
  __device__ static __forceinline__ void compute(const Wt &W, const Act &A, int tl, int kc,
                                                 uint32_t *rec) {
    /* the zero is produced here, behind the loads: without it the compiler decodes each
     * 16-bit value right behind its load, and the loads after that one wait for it */
    const uint32_t late = hipq_late_zero();
    const int un = kc >> 5;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = tl + i * T;
      const uint4 q = W.q[i];
      const float d = hipq_h2f((uint16_t)(W.d[i] | late));
      const uint32_t lo[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
      const uint32_t hi[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                              (q.w >> 4) & HIPQ_M4};
#pragma unroll
      for (int r = 0; r < R; ++r) {
        /* weights are nibble - 8 */
        const uint32_t meta = A.meta[i][r] | late;
        const int bsum = (int)(int16_t)(meta >> 16);
        const int isum = hipq_dot16(lo, A.a0[i][r]) + hipq_dot16(hi, A.a1[i][r]) - 8 * bsum;
        float2 v;
        v.x = (float)isum;
        v.y = d * hipq_h2f((uint16_t)(meta & 0xffff));
        if (u < un) *(float2 *)(rec + r * PER + 2 * u) = v;
      }
    }
  }
};

/* ---- Q4_K ----------------------------------------------------------------------- */
/* A unit is one sub-block: its 16 bytes (eight weights per dword). Consecutive lanes
 * take consecutive sub-blocks, so one load instruction of a wavefront covers 1 KB of
 * consecutive bytes (lanes 32 bytes apart, each taking a sub-block pair with two
 * loads, stream measurably slower). 8 consecutive lanes hold one super-block; its
 * integer sums meet in three DPP steps. */
template <int T, int R, bool PW, int KC> struct GemvQ4K {
  static_assert(T % 8 == 0, "a super-block's eight sub-blocks sit in eight consecutive lanes");
  static constexpr int MAXU = GemvUnits<HIPQ_Q4_K, T, KC>::MAXU;
  static constexpr int PER = GemvRec<HIPQ_Q4_K, PW>::PER_CHUNK;
  struct Act {
    uint4 l[MAXU][R], h[MAXU][R]; /* digits of the sub-block's activations */
    int bs[MAXU][R];              /* the two int16 sums of its halves, as loaded */
    float dA[MAXU][R];
  };
  struct Wt {
    uint4 q[MAXU];
    uint4 hd[MAXU];
  };
  __device__ static __forceinline__ void load_act(Act &A, const QView &qa, const int (&arow)[R],
                                                  int tl, int k0, int kc) {
    const int nsb = qa.K >> 8, un = kc >> 5, b0 = k0 >> 8;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = min(tl + i * T, un - 1);
      const int b = u >> 3, j = u & 7;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const size_t off = (size_t)arow[r] * (qa.K >> 1) + (size_t)(b0 + b) * 128 + j * 16;
        A.l[i][r] = *(const uint4 *)(qa.ql + off);
        A.h[i][r] = *(const uint4 *)(qa.qh + off);
        const int bsw = *(const int *)(qa.bsum + (size_t)arow[r] * (qa.K >> 4) + (b0 + b) * 16 + 2 * j);
        A.bs[i][r] = bsw;
        A.dA[i][r] = qa.d[(size_t)arow[r] * nsb + b0 + b];
      }
    }
  }
  __device__ static __forceinline__ void load_w(Wt &W, const WView &w, int row, int tl, int k0,
                                                int kc) {
    const int nsb = w.K >> 8, un = kc >> 5, b0 = k0 >> 8;
    const uint4 *qs = (const uint4 *)(w.qs + (size_t)row * (w.K >> 1) + (size_t)b0 * 128);
    const uint4 *hdr = (const uint4 *)w.hdr + (size_t)row * nsb + b0;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = min(tl + i * T, un - 1);
      W.q[i] = hipq_ld_stream(qs + u);
      W.hd[i] = hipq_ld_global(hdr + (u >> 3));
    }
  }
  __device__ static __forceinline__ void compute(const Wt &W, const Act &A, int tl, int kc,
                                                 uint32_t *rec) {
    const int un = kc >> 5;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = tl + i * T;
      const bool on = u < un;
      const int uc = on ? u : un - 1;
      const int b = uc >> 3, j = uc & 7;
      const uint4 hd = W.hd[i];
      /* scale and min of sub-block j: byte j of (y, z) holds sc_j and, in its top two
       * bits, m_j >> 4; byte j & 3 of w holds m_j & 15 in its low (j < 4) or high nibble */
      const uint32_t yz = (j < 4 ? hd.y : hd.z) >> (8 * (j & 3));
      const int sc = (int)(yz & 0x3fu);
      const int mn = (int)(((hd.w >> (8 * (j & 3) + (j & 4))) & 0x0fu) | ((yz >> 2) & 0x30u));
      const float dw = hipq_h2f((uint16_t)(hd.x & 0xffff));
      const float dmin = hipq_h2f((uint16_t)(hd.x >> 16));
#pragma unroll
      for (int r = 0; r < R; ++r) {
        int I = __mul24(sc, hipq_dot32_u4(W.q[i], A.l[i][r], A.h[i][r]));
        int Im = __mul24(mn, (int)(int16_t)(A.bs[i][r] & 0xffff) + (A.bs[i][r] >> 16));
        I += hipq_dpp_i<HIPQ_DPP_XOR1>(I); /* the sub-block pair */
        Im += hipq_dpp_i<HIPQ_DPP_XOR1>(Im);
        if (PW) {
          if (on && (j & 1) == 0) {
            uint32_t *o = rec + r * PER + b * 10;
            o[j >> 1] = (uint32_t)I;
            o[4 + (j >> 1)] = (uint32_t)Im;
            if (j == 0) {
              o[8] = __float_as_uint(dw * A.dA[i][r]);
              o[9] = __float_as_uint(dmin * A.dA[i][r]);
            }
          }
        } else {
          I += hipq_dpp_i<HIPQ_DPP_XOR2>(I); /* the four pairs of the super-block */
          Im += hipq_dpp_i<HIPQ_DPP_XOR2>(Im);
          I += hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(I);
          Im += hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(Im);
          if (on && j == 0) {
            float4 v;
            v.x = (float)I;
            v.y = dw * A.dA[i][r];
            v.z = (float)Im;
            v.w = dmin * A.dA[i][r];
            *(float4 *)(rec + r * PER + b * 4) = v;
          }
        }
      }
    }
  }
};

/* ---- Q6_K ----------------------------------------------------------------------- */
/* A unit is 64 weights = 16 B of each ql plane + 16 B of qh, unit uu = half*2 + hl of
 * a super-block. Dword t of the unit belongs to partial l = hl*4 + t; lanes uu and
 * uu^2 hold the two 128-element halves. */
template <int T, int R, bool PW, int KC> struct GemvQ6K {
  static constexpr int MAXU = GemvUnits<HIPQ_Q6_K, T, KC>::MAXU;
  static constexpr int PER = GemvRec<HIPQ_Q6_K, PW>::PER_CHUNK;
  struct Act {
    int4 a[MAXU][R][4];
    float dA[MAXU][R];
  };
  struct Wt {
    uint4 qa[MAXU], qb[MAXU], qh[MAXU];
    int scw[MAXU];
    uint16_t d[MAXU];
  };
  __device__ static __forceinline__ void load_act(Act &A, const QView &qa, const int (&arow)[R],
                                                  int tl, int k0, int kc) {
    const int nsb = qa.K >> 8, un = kc >> 6, b0 = k0 >> 8;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = min(tl + i * T, un - 1);
      const int b = u >> 2, uu = u & 3, half = uu >> 1, hl = uu & 1;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int8_t *ab =
          qa.q + (size_t)arow[r] * qa.K + (size_t)(b0 + b) * 256 + half * 128 + hl * 16;
#pragma unroll
        for (int g = 0; g < 4; ++g) A.a[i][r][g] = *(const int4 *)(ab + 32 * g);
        A.dA[i][r] = qa.d[(size_t)arow[r] * nsb + b0 + b];
      }
    }
  }
  __device__ static __forceinline__ void load_w(Wt &W, const WView &w, int row, int tl, int k0,
                                                int kc) {
    const int nsb = w.K >> 8, b0 = k0 >> 8, un = kc >> 6;
    /* two ql planes of N * K / 4 bytes each: a unit's first and second 16 bytes */
    const uint8_t *qlrow = w.qs + (size_t)row * (w.K >> 2) + (size_t)b0 * 64;
    const uint8_t *qlrow2 = qlrow + (size_t)w.N * (w.K >> 2);
    const uint8_t *qhrow = w.qh + (size_t)row * (w.K >> 2) + (size_t)b0 * 64;
    const int8_t *scrow = w.sc + (size_t)row * (w.K >> 4) + (size_t)b0 * 16;
    const uint16_t *drow = w.d + (size_t)row * nsb + b0;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = min(tl + i * T, un - 1);
      const int b = u >> 2;
      /* consecutive lanes take consecutive 16-byte pieces of every plane */
      W.qa[i] = hipq_ld_stream((const uint4 *)(qlrow + u * 16));
      W.qb[i] = hipq_ld_stream((const uint4 *)(qlrow2 + u * 16));
      W.qh[i] = hipq_ld_stream((const uint4 *)(qhrow + u * 16));
      W.scw[i] = hipq_ld_global((const int *)(scrow + u * 4));
      W.d[i] = hipq_ld_global(drow + b);
    }
  }
  __device__ static __forceinline__ void compute(const Wt &W, const Act &A, int tl, int kc,
                                                 uint32_t *rec) {
    const int un = kc >> 6;
#pragma unroll
    for (int i = 0; i < MAXU; ++i) {
      if (i * T >= un) break;
      const int u = tl + i * T;
      const bool on = u < un;
      const int uc = on ? u : un - 1;
      const int b = uc >> 2, uu = uc & 3, half = uu >> 1, hl = uu & 1;
      const uint32_t QA[4] = {W.qa[i].x, W.qa[i].y, W.qa[i].z, W.qa[i].w};
      const uint32_t QB[4] = {W.qb[i].x, W.qb[i].y, W.qb[i].z, W.qb[i].w};
      const uint32_t H[4] = {W.qh[i].x, W.qh[i].y, W.qh[i].z, W.qh[i].w};
      const int scw = W.scw[i];
      const int s0 = (int)(int8_t)(scw & 0xff), s1 = (int)(int8_t)((scw >> 8) & 0xff);
      const int s2 = (int)(int8_t)((scw >> 16) & 0xff), s3 = (int)(int8_t)((scw >> 24) & 0xff);
      const float dwt = hipq_h2f(W.d[i]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int a0w[4] = {A.a[i][r][0].x, A.a[i][r][0].y, A.a[i][r][0].z, A.a[i][r][0].w};
        const int a1w[4] = {A.a[i][r][1].x, A.a[i][r][1].y, A.a[i][r][1].z, A.a[i][r][1].w};
        const int a2w[4] = {A.a[i][r][2].x, A.a[i][r][2].y, A.a[i][r][2].z, A.a[i][r][2].w};
        const int a3w[4] = {A.a[i][r][3].x, A.a[i][r][3].y, A.a[i][r][3].z, A.a[i][r][3].w};
        int P[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          /* 6-bit values of the four 32-element groups, 4 at a time;
           * (q6 - 32) . a = q6 . a - 32 . a, both via v_dot4 */
          const int v0 = (int)((QA[t] & HIPQ_M4) | ((H[t] << 4) & 0x30303030u));
          const int v1 = (int)((QB[t] & HIPQ_M4) | ((H[t] << 2) & 0x30303030u));
          const int v2 = (int)(((QA[t] >> 4) & HIPQ_M4) | (H[t] & 0x30303030u));
          const int v3 = (int)(((QB[t] >> 4) & HIPQ_M4) | ((H[t] >> 2) & 0x30303030u));
          const int c32 = 0x20202020;
          int p = __mul24(s0, hipq_dot4(v0, a0w[t], 0) - hipq_dot4(c32, a0w[t], 0));
          p += __mul24(s1, hipq_dot4(v1, a1w[t], 0) - hipq_dot4(c32, a1w[t], 0));
          p += __mul24(s2, hipq_dot4(v2, a2w[t], 0) - hipq_dot4(c32, a2w[t], 0));
          p += __mul24(s3, hipq_dot4(v3, a3w[t], 0) - hipq_dot4(c32, a3w[t], 0));
          P[t] = p + hipq_dpp_i<HIPQ_DPP_XOR2>(p); /* both 128-element halves */
        }
        if (on && half == 0) {
          uint32_t *o = rec + r * PER + b * 9;
#pragma unroll
          for (int t = 0; t < 4; ++t) o[hl * 4 + t] = (uint32_t)P[t];
          if (hl == 0) o[8] = __float_as_uint(A.dA[i][r] * dwt);
        }
      }
    }
  }
};

template <int DT, int T, int R, bool PW, int KC> struct GemvFmt;
template <int T, int R, bool PW, int KC> struct GemvFmt<HIPQ_Q4_0, T, R, PW, KC> { typedef GemvQ40<T, R, PW, KC> type; };
template <int T, int R, bool PW, int KC> struct GemvFmt<HIPQ_Q4_K, T, R, PW, KC> { typedef GemvQ4K<T, R, PW, KC> type; };
template <int T, int R, bool PW, int KC> struct GemvFmt<HIPQ_Q6_K, T, R, PW, KC> { typedef GemvQ6K<T, R, PW, KC> type; };

/* ---- engine --------------------------------------------------------------------- */

struct GemvOut {
  float v;    /* finished output                                   */
  int g, r;   /* weight row within the group, activation row index */
  bool valid; /* this lane carries an output                       */
};

/**
 * Computes, for the G weight rows starting at row0 (clamped to the matrix) and
 * the R activation rows arow[], all G*R outputs. Must be called by every lane
 * of every wavefront of the workgroup (it uses __syncthreads); `lds` is this
 * wavefront's private region of G*R*PER_CHUNK dwords. With PW, activation rows
 * arow[r] < pair_rows use the per-sub-block-pair order (Q4_K only).
 */
/* The records are private to one wavefront. Its lanes run in lockstep, so LDS
 * stores only have to be complete before other lanes read them: no workgroup
 * barrier, and the wavefronts of a workgroup stay free to drift apart (one
 * streams weights while another computes). */
__device__ __forceinline__ void hipq_wave_lds_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
}

/* The pieces of the engine, so that callers with several weight-row groups per
 * wavefront can keep the loads of the next group in flight while this one is
 * computed (see gemv_engine for the plain sequence). */
template <int DT, int T, int R, int G, bool PW, int KC = HIPQ_KCHUNK> struct GemvCore {
  typedef typename GemvFmt<DT, T, R, PW, KC>::type F;
  typedef typename F::Act Act;
  static constexpr int RW = 64 / T; /* weight rows streamed at once */
  static constexpr int NP = G / RW; /* passes per group */
  static constexpr int PER = GemvRec<DT, PW>::PER_CHUNK;
  static constexpr int LPO = GemvRec<DT, PW>::LANES_PER_OUT;
  static_assert(G % RW == 0, "group must be a multiple of the rows streamed at once");
  static_assert(G * R * LPO <= 64, "one lane per fp32 chain");
  struct Wts {
    typename F::Wt W[NP];
  };
  /* the fp32 chain this lane runs in phase 2 */
  struct Chain {
    int cg, cr, l;
    bool on, pairwise;
    float acc, accm;
  };

  __device__ static __forceinline__ void load_act(Act &A, const QView &qa, const int (&arow)[R],
                                                  int k0, int kc) {
    F::load_act(A, qa, arow, (threadIdx.x & 63) % T, k0, kc);
  }
  /* issue the loads of the G weight rows from row0 (clamped to the matrix); P0, P1: of passes P0 .. P1 - 1 only */
  template <int P0 = 0, int P1 = NP>
  __device__ static __forceinline__ void load_w(Wts &w, const WView &wv, int row0, int k0, int kc) {
    const int lane = threadIdx.x & 63, tl = lane % T;
#pragma unroll
    for (int pass = P0; pass < P1; ++pass) {
      const int g = pass * RW + lane / T;
      F::load_w(w.W[pass], wv, min(row0 + g, wv.N - 1), tl, k0, kc);
    }
  }
  /* phase 1: integer partial sums of this chunk into the wavefront's LDS records */
  __device__ static __forceinline__ void compute(const Wts &w, const Act &A, int kc, uint32_t *lds) {
    const int lane = threadIdx.x & 63, tl = lane % T;
#pragma unroll
    for (int pass = 0; pass < NP; ++pass) {
      const int g = pass * RW + lane / T;
      F::compute(w.W[pass], A, tl, kc, lds + g * R * PER);
    }
  }
  __device__ static __forceinline__ Chain begin(const int (&arow)[R], int pair_rows) {
    const int lane = threadIdx.x & 63;
    Chain c;
    const int ci = lane / LPO;
    c.l = lane % LPO;
    c.on = ci < G * R;
    c.cg = c.on ? ci / R : 0;
    c.cr = c.on ? ci % R : 0;
    c.acc = 0.f;
    c.accm = 0.f;
    c.pairwise = false;
    if (PW) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (r == c.cr) c.pairwise = arow[r] < pair_rows;
    }
    return c;
  }
  /* phase 2: this lane's fp32 chain over the records of one chunk, reference order */
  __device__ static __forceinline__ void chain(Chain &c, int kc, const uint32_t *lds) {
    const uint32_t *crec = lds + (c.cg * R + c.cr) * PER;
    const bool chain = c.on, pairwise = c.pairwise;
    const int l = c.l;
    float acc = c.acc, accm = c.accm;
    (void)pairwise;
    (void)l;
    if (chain) {
      if (DT == HIPQ_Q4_0) {
        const int nb = kc >> 5;
#pragma unroll 4
        for (int b = 0; b < nb; ++b) {
          const float2 v = *(const float2 *)(crec + 2 * b);
          acc = fmaf(v.x, v.y, acc);
        }
      } else if (DT == HIPQ_Q4_K && !PW) {
        const int nb = kc >> 8;
#pragma unroll 4
        for (int b = 0; b < nb; ++b) {
          const float4 v = *(const float4 *)(crec + 4 * b);
          acc = fmaf(v.x, v.y, acc);
          accm = fmaf(v.z, v.w, accm);
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
#pragma unroll 4
        for (int b = 0; b < nb; ++b) {
          const uint32_t *o = crec + b * 9;
          acc = fmaf(__uint_as_float(o[8]), (float)(int)o[l], acc);
        }
      }
    }
    c.acc = acc;
    c.accm = accm;
  }
  __device__ static __forceinline__ GemvOut finish(const Chain &c) {
    const bool chain = c.on;
    const int cg = c.cg, cr = c.cr, l = c.l;
    const float acc = c.acc, accm = c.accm;
    (void)l;
    (void)accm;
  GemvOut out;
  out.g = cg;
  out.r = cr;
  if (DT == HIPQ_Q4_K) {
    out.v = acc - accm;
    out.valid = chain;
  } else if (DT == HIPQ_Q6_K) {
    /* ((a0+a4)+(a2+a6)) + ((a1+a5)+(a3+a7)) */
    float v = acc;
    /* lane l of the eight takes lanes l + 4, l + 2, l + 1 in turn (row_shl): for l = 0, the only one
     * stored, the sums of the exchange with lanes l ^ 4, l ^ 2, l ^ 1, without the LDS crossbar */
    v = v + hipq_dpp_f<0x104>(v);
    v = v + hipq_dpp_f<0x102>(v);
    v = v + hipq_dpp_f<0x101>(v);
    out.v = v;
    out.valid = chain && l == 0;
  } else {
    out.v = acc;
    out.valid = chain;
  }
  return out;
  }
};

template <int DT, int T, int R, int G, bool PW, int KC = HIPQ_KCHUNK, int FK = 0>
__device__ __forceinline__ GemvOut gemv_engine(const WView &w, int row0, const QView &qa,
                                               const int (&arow)[R], int pair_rows,
                                               uint32_t *lds) {
  typedef GemvCore<DT, T, R, G, PW, KC> E;
  typename E::Chain c = E::begin(arow, pair_rows);
  if constexpr (FK != 0) {
    /* FK: the row length, where the launcher has seen one of the usual ones (one chunk). With it a constant no
     * load sits behind a condition and the waits can count them: the activations' loads first, nothing moved
     * across, then the weights', and each pass over the weight rows waits for its own loads only. */
    typename E::Act A;
    E::load_act(A, qa, arow, 0, FK);
    __builtin_amdgcn_sched_barrier(0);
    typename E::Wts W;
    E::load_w(W, w, row0, 0, FK);
    __builtin_amdgcn_sched_barrier(0);
    E::compute(W, A, FK, lds);
    hipq_wave_lds_sync();
    E::chain(c, FK, lds);
    hipq_wave_lds_sync();
    return E::finish(c);
  }
  auto chunk = [&](int k0, int kc) {
    /* the weights first: the activations' loads are followed by arithmetic on what
     * they return, and in the other order the weight loads would be issued only
     * after that round trip */
    typename E::Wts W;
    E::load_w(W, w, row0, k0, kc);
    typename E::Act A;
    E::load_act(A, qa, arow, k0, kc);
    E::compute(W, A, kc, lds);
    hipq_wave_lds_sync();
    E::chain(c, kc, lds);
    hipq_wave_lds_sync();
  };
  /* Rows of one chunk (the usual case) run outside the loop: inside it the compiler
   * guards every load's destination registers against the loads of the previous
   * iteration, which serialises the loads of the first one as well. */
  if (w.K <= KC) {
    chunk(0, w.K);
  } else {
    for (int k0 = 0; k0 < w.K; k0 += KC) chunk(k0, min(KC, w.K - k0));
  }
  return E::finish(c);
}

/* LDS dwords one wavefront needs for G weight rows x R activation rows. */
template <int DT, int R, int G, bool PW> struct GemvLds {
  static constexpr int DWORDS = G * R * GemvRec<DT, PW>::PER_CHUNK;
};

#endif /* HIPQ_GEMV_DEVICE_H */
