// SPDX-License-Identifier: Apache-2.0
/**
 * @file   quantize_device.h
 * @brief  The Q8_K activation quantizer of one wavefront (one 256-value
 *         super-block) and the Q8_0 quantizer of eight lanes (one 32-value
 *         block), shared by the quantizer kernels and by kernels that quantize
 *         rows as part of another launch.
 *
 * Bit-exact with the reference CPU quantizers in an x86 AVX2 GCC build
 * (IMPL = nntrainer/tensor/cpu_backend/ggml_interface/nntr_ggml_impl):
 *   Q8_0 IMPL/nntr_ggml_impl_quant.cpp:613-701 and the per-row content of
 *        IMPL/nntr_ggml_impl.cpp:7879-7980
 *   ROW  IMPL/nntr_ggml_impl_quant.cpp:1334-1374, where the compiler fuses
 *        iscale*x + 1.5*2^23 into a single rounding
 *   MAT  IMPL/nntr_ggml_impl.cpp:7504-7737 (product rounded to fp32, then to
 *        the nearest-even integer; scale negative iff some x == +amax)
 */
#ifndef HIPQ_QUANTIZE_DEVICE_H
#define HIPQ_QUANTIZE_DEVICE_H
#include "hipq_internal.h"

static constexpr float kRoundMagic = 12582912.f; /* 1.5 * 2^23 */

__device__ __forceinline__ int magic_to_int(float biased) {
  return (int)(__float_as_uint(biased) & 0x007fffffu) - 0x00400000;
}

__device__ __forceinline__ int pack4(int a, int b, int c, int d) {
  return (a & 0xff) | ((b & 0xff) << 8) | ((c & 0xff) << 16) | ((d & 0xff) << 24);
}

/* The 16-byte matrix operand of a 16-value group, from the four lanes of a quad that
 * hold its values 4i .. 4i+3 each (q[0..3] of lane i): the 8 even values first, then
 * the 8 odd ones. Every lane of the quad returns the whole operand. */
__device__ __forceinline__ uint4 hipq_quad_operand(const int (&q)[4]) {
  const int mine = (q[0] & 0xff) | ((q[2] & 0xff) << 8) | ((q[1] & 0xff) << 16) | ((q[3] & 0xff) << 24);
  const uint32_t d0 = (uint32_t)hipq_dpp_i<0x00>(mine), d1 = (uint32_t)hipq_dpp_i<0x55>(mine);
  const uint32_t d2 = (uint32_t)hipq_dpp_i<0xAA>(mine), d3 = (uint32_t)hipq_dpp_i<0xFF>(mine);
  return make_uint4((d0 & 0xffffu) | (d1 << 16), (d2 & 0xffffu) | (d3 << 16), (d0 >> 16) | (d1 & 0xffff0000u),
                    (d2 >> 16) | (d3 & 0xffff0000u));
}

/* Q8_0: the calling lane holds four consecutive values of a 32-value block, the
 * eight lanes of the block are consecutive. Returns the lane's four int8 values
 * packed; dh = the block's fp16 scale. */
__device__ __forceinline__ int hipq_quantize_q8_0_lane(const float4 &x, uint16_t &dh, int &qsum) {
  float amax = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
  amax = hipq_group_max<8>(amax);
  const float d = __fdiv_rn(amax, 127.f);
  const float id = (amax != 0.0f) ? __fdiv_rn(127.f, amax) : 0.0f;
  const int q0 = (int)rintf(__fmul_rn(x.x, id));
  const int q1 = (int)rintf(__fmul_rn(x.y, id));
  const int q2 = (int)rintf(__fmul_rn(x.z, id));
  const int q3 = (int)rintf(__fmul_rn(x.w, id));
  dh = hipq_f2h(d);
  qsum = q0 + q1 + q2 + q3;
  return pack4(q0, q1, q2, q3);
}

/* output forms of the Q8_K quantizer */
enum {
  Q8K_PLANES = 0,
  Q8K_CANONICAL = 1,
  Q8K_ROWMMA = 3,
  Q8K_DIGITS = 4, /* of the planes only what the Q4_K GEMV reads: ql, qh, bsum, d */
  Q8K_BYTES = 5   /* of the planes only what the Q6_K GEMV reads: q, d */
};

/* Super-block sb = (row m, block b) by the calling wavefront (all 64 lanes), lane l
 * holding its values 4l .. 4l+3 in xv. Rows below mat_rows take the 4-row
 * quantizer's semantics, the others the row quantizer's. d_stride: distance of
 * consecutive super-blocks' scales in d_out (the row form only). */
template <int MODE>
__device__ __forceinline__ void hipq_quantize_q8_K_values(
  const float4 &xv, int64_t m, int b, int64_t sb, int nsb, int64_t mat_rows, int8_t *__restrict__ q_out,
  float *__restrict__ d_out, int16_t *__restrict__ bsum_out, uint8_t *__restrict__ canon_out,
  uint16_t *__restrict__ amin_out, uint16_t *__restrict__ ql_out, uint16_t *__restrict__ qh_out,
  int d_stride = 1) {
  const int lane = threadIdx.x & 63;
  const float x[4] = {xv.x, xv.y, xv.z, xv.w};

  float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
  amax = hipq_wave_max(amax); /* the same value in every lane, without an exchange through LDS */

  int q[4];
  float d;
  if (amax == 0.0f) {
    q[0] = q[1] = q[2] = q[3] = 0;
    d = 0.f;
  } else if (m < mat_rows) {
    /* 4-row quantizer semantics */
    const bool hit = (x[0] == amax) | (x[1] == amax) | (x[2] == amax) | (x[3] == amax);
    const bool pos_hit = __ballot(hit) != 0ull;
    const float iscale = pos_hit ? __fdiv_rn(-127.f, amax) : __fdiv_rn(127.f, amax);
    d = __fdiv_rn(1.f, iscale);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int v = (int)rintf(__fmul_rn(x[i], iscale));
      q[i] = max(-128, min(127, v));
    }
  } else {
    /* row quantizer semantics: sign of the FIRST element of maximal magnitude */
    float cand = 0.f;
    bool has = false;
#pragma unroll
    for (int i = 3; i >= 0; --i)
      if (fabsf(x[i]) == amax) {
        cand = x[i];
        has = true;
      }
    const unsigned long long mask = __ballot(has);
    const int first = __ffsll((long long)mask) - 1;
    const float vmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cand), first));
    const float iscale = __fdiv_rn(-127.f, vmax);
    d = __fdiv_rn(1.f, iscale);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      q[i] = min(127, magic_to_int(__fmaf_rn(iscale, x[i], kRoundMagic)));
  }

  const int packed = pack4(q[0], q[1], q[2], q[3]);
  int gsum = q[0] + q[1] + q[2] + q[3];
  gsum = hipq_group_sum_i<4>(gsum); /* 4 lanes = one 16-value group */

  if (MODE == Q8K_CANONICAL) {
    uint8_t *o = canon_out + sb * 292;
    if (lane == 0) *(float *)o = d;
    *(int *)(o + 4 + lane * 4) = packed;
    if ((lane & 3) == 0) *(int16_t *)(o + 260 + (lane >> 2) * 2) = (int16_t)gsum;
  } else if (MODE == Q8K_ROWMMA) {
    /* row-major, each 16-value group stored as its 8 even then its 8 odd values:
     * this lane's four values are elements 4l .. 4l+3 of group lane / 4 */
    const uint4 op = hipq_quad_operand(q);
    if ((lane & 3) == 0) *(uint4 *)(q_out + sb * 256 + (lane >> 2) * 16) = op;
    if (lane == 0) d_out[sb * d_stride] = d;
    const int bs = gsum + hipq_dpp_i<0x104>(gsum); /* row_shl:4: lane l takes lane l + 4; two 16-value groups = one sub-block (read in lanes 0 and 8 of a row) */
    if ((lane & 7) == 0) {
      const int l6 = bs & 63;
      amin_out[sb * 16 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)l6));
      amin_out[sb * 16 + 8 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)(bs - l6)));
    }
  } else {
    if (MODE != Q8K_DIGITS) *(int *)(q_out + sb * 256 + lane * 4) = packed;
    if (lane == 0) d_out[sb] = d;
    if (MODE != Q8K_BYTES) {
      if ((lane & 3) == 0) bsum_out[sb * 16 + (lane >> 2)] = (int16_t)gsum;
      /* 4-bit digits for the v_dot8_u32_u4 kernels: q = 16 * (qh - 8) + ql */
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo |= (uint32_t)(q[i] & 15) << (4 * i);
        hi |= (uint32_t)(((q[i] >> 4) + 8) & 15) << (4 * i);
      }
      ql_out[sb * 64 + lane] = (uint16_t)lo;
      qh_out[sb * 64 + lane] = (uint16_t)hi;
    }
  }
}

/* The same with the values read from row m of A (rows M and beyond read as zeros). */
template <int MODE>
__device__ __forceinline__ void hipq_quantize_q8_K_wave(
  const float *__restrict__ A, int64_t M, int64_t sb, int nsb, int64_t lda, int64_t mat_rows,
  int8_t *__restrict__ q_out, float *__restrict__ d_out, int16_t *__restrict__ bsum_out,
  uint8_t *__restrict__ canon_out, uint16_t *__restrict__ amin_out, uint16_t *__restrict__ ql_out,
  uint16_t *__restrict__ qh_out) {
  const int lane = threadIdx.x & 63;
  const int64_t m = sb / nsb;
  const int b = (int)(sb - m * nsb);
  float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (m < M) xv = *(const float4 *)(A + m * lda + (int64_t)b * 256 + lane * 4);
  hipq_quantize_q8_K_values<MODE>(xv, m, b, sb, nsb, mat_rows, q_out, d_out, bsum_out, canon_out, amin_out,
                                  ql_out, qh_out);
}

#endif /* HIPQ_QUANTIZE_DEVICE_H */
