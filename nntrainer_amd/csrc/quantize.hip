// SPDX-License-Identifier: Apache-2.0
/**
 * @file   quantize.hip
 * @brief  Activation quantizers fp32 -> Q8_0 / Q8_K for gfx950.
 *
 * Bit-exact with the reference CPU quantizers in an x86 AVX2 GCC build
 * (paths relative to the reference checkout, IMPL =
 * nntrainer/tensor/cpu_backend/ggml_interface/nntr_ggml_impl):
 *   Q8_0      IMPL/nntr_ggml_impl_quant.cpp:613-701 and the per-row content of
 *             IMPL/nntr_ggml_impl.cpp:7879-7980
 *   Q8_K ROW  IMPL/nntr_ggml_impl_quant.cpp:1334-1374, where the compiler fuses
 *             iscale*x + 1.5*2^23 into a single rounding
 *   Q8_K MAT  IMPL/nntr_ggml_impl.cpp:7504-7737 (product rounded to fp32, then
 *             to the nearest-even integer; scale negative iff some x == +amax)
 * Every floating-point step that decides a bit is an explicit round-to-nearest
 * intrinsic (__fdiv_rn, __fmul_rn, __fmaf_rn, rintf), so the compiler can
 * neither contract nor approximate it.
 *
 * Work mapping: Q8_0 uses 8 lanes per 32-value block (one 128-bit load per
 * lane, 8 blocks per wavefront); Q8_K uses one wavefront per 256-value
 * super-block (one 128-bit load per lane). Reductions run over DPP.
 */
#include "quantize_device.h"

namespace {

/* ---- Q8_0 ---------------------------------------------------------------- */
template <bool CANONICAL>
__global__ __launch_bounds__(256) void quantize_q8_0_kernel(
  const float *__restrict__ A, int64_t n_blocks_total, int nb, int64_t lda,
  int8_t *__restrict__ q_out, uint32_t *__restrict__ meta_out,
  uint8_t *__restrict__ canon_out) {
  const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t blk = gtid >> 3;
  const int sub = (int)(gtid & 7);
  const bool live = blk < n_blocks_total;
  if (!live) blk = n_blocks_total - 1; /* keep the lane in the reductions */
  const int64_t m = blk / nb;
  const int b = (int)(blk - m * nb);
  const float4 x = *(const float4 *)(A + m * lda + (int64_t)b * 32 + sub * 4);

  uint16_t dh;
  int qsum;
  const int packed = hipq_quantize_q8_0_lane(x, dh, qsum);

  if (CANONICAL) {
    if (!live) return;
    uint8_t *o = canon_out + blk * 34;
    if (sub == 0) *(uint16_t *)o = dh;
    uint16_t *qs = (uint16_t *)(o + 2 + sub * 4);
    qs[0] = (uint16_t)(packed & 0xffff);
    qs[1] = (uint16_t)((unsigned)packed >> 16);
  } else {
    int bsum = hipq_group_sum_i<8>(qsum);
    if (!live) return;
    *(int *)(q_out + (m * nb + b) * 32 + sub * 4) = packed;
    if (sub == 0) meta_out[m * nb + b] = (uint32_t)dh | ((uint32_t)(bsum & 0xffff) << 16);
  }
}

/* ---- Q8_K ---------------------------------------------------------------- */

/* One wavefront per (row, super-block). */
template <int MODE>
__global__ __launch_bounds__(256) void quantize_q8_K_kernel(
  const float *__restrict__ A, int64_t M, int64_t n_sb_total, int nsb, int64_t lda,
  int64_t mat_rows, int8_t *__restrict__ q_out, float *__restrict__ d_out,
  int16_t *__restrict__ bsum_out, uint8_t *__restrict__ canon_out,
  uint16_t *__restrict__ amin_out, uint16_t *__restrict__ ql_out, uint16_t *__restrict__ qh_out) {
  const int64_t sb = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (sb >= n_sb_total) return; /* uniform per wavefront */
  hipq_quantize_q8_K_wave<MODE>(A, M, sb, nsb, lda, mat_rows, q_out, d_out, bsum_out, canon_out, amin_out,
                                ql_out, qh_out);
}

/* The tiled form for the Q4_K prefill GEMM. A wavefront takes super-block b of four
 * consecutive rows (a 4-aligned quad, so that all four follow the same quantizer's
 * semantics): sixteen lanes per row, sixteen values per lane in four 16-byte loads, lane
 * l of a row holding values 64 i + 4 l .. + 3 of the super-block from load i. That is the
 * arithmetic of hipq_quantize_q8_K_values value by value; the reductions stay inside a
 * 16-lane row (four DPP steps) and the scale's two divisions serve sixteen values per
 * lane instead of four. Rows M and beyond of the last 128-row tile are written as zeros. */
__global__ __launch_bounds__(256) void quantize_q8_K_tiled_kernel(
  const float *__restrict__ A, int64_t M, int64_t n_units, int nsb, int64_t lda, int64_t mat_rows,
  int8_t *__restrict__ q_out, float *__restrict__ d_out, uint16_t *__restrict__ amin_out) {
  const int64_t unit = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= n_units) return; /* uniform per wavefront */
  const int lane = threadIdx.x & 63, l16 = lane & 15;
  const int64_t mq = unit / nsb;
  const int b = (int)(unit - mq * nsb);
  const int64_t m = mq * 4 + (lane >> 4);
  float x[4][4];
  /* the four loads at once and unconditionally (a row past M reads the last one and is zeroed after): behind a
   * condition they went out two at a time, each pair a round trip of its own */
  const float *src = A + (m < M ? m : M - 1) * lda + (int64_t)b * 256 + 4 * l16;
  float4 v4[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) v4[i] = *(const float4 *)(src + 64 * i);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float4 v = m < M ? v4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    x[i][0] = v.x, x[i][1] = v.y, x[i][2] = v.z, x[i][3] = v.w;
  }
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int c = 0; c < 4; ++c) amax = fmaxf(amax, fabsf(x[i][c]));
  amax = hipq_group_max<16>(amax);
  const bool zero = amax == 0.0f;
  const float amax1 = zero ? 1.f : amax; /* keeps the arithmetic below finite; the results are dropped */
  int q[4][4];
  float d;
  if (mq * 4 < mat_rows) { /* uniform: the 4-row quantizer's semantics */
    bool hit = false;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) hit = hit | (x[i][c] == amax);
    const unsigned row_hits = (unsigned)(__ballot(hit) >> (lane & 48)) & 0xffffu;
    const float iscale = row_hits ? __fdiv_rn(-127.f, amax1) : __fdiv_rn(127.f, amax1);
    d = __fdiv_rn(1.f, iscale);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int v = (int)rintf(__fmul_rn(x[i][c], iscale));
        q[i][c] = max(-128, min(127, v));
      }
  } else { /* the row quantizer's: sign of the FIRST value of maximal magnitude */
    float cand = 0.f;
    int key = 1024;
#pragma unroll
    for (int i = 3; i >= 0; --i)
#pragma unroll
      for (int c = 3; c >= 0; --c)
        if (fabsf(x[i][c]) == amax) {
          cand = x[i][c];
          key = 64 * i + 4 * l16 + c;
        }
    int kmin = key;
    kmin = min(kmin, hipq_dpp_i<HIPQ_DPP_XOR1>(kmin));
    kmin = min(kmin, hipq_dpp_i<HIPQ_DPP_XOR2>(kmin));
    kmin = min(kmin, hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(kmin));
    kmin = min(kmin, hipq_dpp_i<HIPQ_DPP_MIRROR>(kmin));
    const unsigned owners = (unsigned)(__ballot(key == kmin) >> (lane & 48)) & 0xffffu;
    const int src = (lane & 48) + __ffs((int)owners) - 1; /* keys are distinct: one owner, or all when none has one */
    const float vmax = __shfl(cand, src, HIPQ_WAVE);
    const float iscale = __fdiv_rn(-127.f, zero ? 1.f : vmax);
    d = __fdiv_rn(1.f, iscale);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) q[i][c] = min(127, magic_to_int(__fmaf_rn(iscale, x[i][c], kRoundMagic)));
  }
  if (zero) {
    d = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i][0] = q[i][1] = q[i][2] = q[i][3] = 0;
  }

  const int64_t mt = m >> 7;
  const int r = (int)(m & 127);
  const int64_t rb = (mt * nsb + b) * 128 + r;
  if (l16 == 0) d_out[rb] = d;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    /* the quad of lanes 4k .. 4k+3 holds the 16-value group 4 i + k: half (k & 1) of
     * sub-block jb = 2 i + (k >> 1). The GEMM's lane (row, g) takes sub-blocks 4g .. 4g+3,
     * two 32-deep steps each: the group is the operand of step st of lane group g. */
    const int jb = 2 * i + (l16 >> 3), g = i >> 1;
    const int st = 2 * (jb & 3) + ((l16 >> 2) & 1);
    const int64_t tile = (mt * (2 * nsb) + b * 2 + (st >> 2)) * 16384;
    const int off = ((r >> 5) * 4 + (st & 3)) * 1024 + (g * 32 + (r & 31)) * 16;
    const uint4 op = hipq_quad_operand(q[i]);
    if ((lane & 3) == 0) *(uint4 *)(q_out + tile + off) = op;
    int bs = q[i][0] + q[i][1] + q[i][2] + q[i][3];
    bs += hipq_dpp_i<HIPQ_DPP_XOR1>(bs);
    bs += hipq_dpp_i<HIPQ_DPP_XOR2>(bs);
    bs += hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(bs); /* the eight lanes of the sub-block */
    if ((lane & 7) == 0) {
      const int l6 = bs & 63;
      amin_out[rb * 16 + jb] = __half_as_ushort(__float2half_rn((float)l6));
      amin_out[rb * 16 + 8 + jb] = __half_as_ushort(__float2half_rn((float)(bs - l6)));
    }
  }
}

} // namespace

namespace hipq {

int launch_quantize_q8_0(const float *A, int64_t M, int64_t K, int64_t lda,
                         const QAct *qa, void *canonical_out, hipStream_t s) {
  if (M <= 0) return HIPQ_OK;
  if (K % 32 || lda < K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q8_0: K=%lld must be a multiple of 32 and lda >= K", (long long)K);
  if (((uintptr_t)A & 15) || (lda & 3))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  const int nb = (int)(K / 32);
  const int64_t total = M * nb;
  const int64_t threads = total * 8;
  const unsigned grid = (unsigned)((threads + 255) / 256);
  if (canonical_out)
    hipq::launch_kernel("quantize_q8_0_kernel<true>", quantize_q8_0_kernel<true>, dim3(grid), dim3(256), 0, s, A, total, nb, lda,
                       nullptr, nullptr, (uint8_t *)canonical_out);
  else
    hipq::launch_kernel("quantize_q8_0_kernel<false>", quantize_q8_0_kernel<false>, dim3(grid), dim3(256), 0, s, A, total, nb, lda,
                       qa->q, qa->meta, nullptr);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_quantize_q8_K(const float *A, int64_t M, int64_t K, int64_t lda,
                         int64_t mat_rows, const QAct *qa, void *canonical_out,
                         hipStream_t s) {
  if (M <= 0) return HIPQ_OK;
  if (K % 256 || lda < K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q8_K: K=%lld must be a multiple of 256 and lda >= K", (long long)K);
  if (((uintptr_t)A & 15) || (lda & 3))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  const int nsb = (int)(K / 256);
  const int64_t total = M * nsb;
  const unsigned grid = (unsigned)((total + 3) / 4);
  if (canonical_out)
    hipq::launch_kernel("quantize_q8_K_kernel<Q8K_CANONICAL>", quantize_q8_K_kernel<Q8K_CANONICAL>, dim3(grid), dim3(256), 0, s, A, M, total,
                       nsb, lda, mat_rows, nullptr, nullptr, nullptr, (uint8_t *)canonical_out, nullptr, nullptr,
                       nullptr);
  else
    hipq::launch_kernel("quantize_q8_K_kernel<Q8K_PLANES>", quantize_q8_K_kernel<Q8K_PLANES>, dim3(grid), dim3(256), 0, s, A, M, total, nsb,
                       lda, mat_rows, qa->q, qa->d, qa->bsum, nullptr, nullptr, (uint16_t *)qa->ql,
                       (uint16_t *)qa->qh);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_quantize_q8_K_rowmma(const float *A, int64_t M, int64_t K, int64_t lda, const QAct *qa,
                                hipStream_t s, int64_t mat_rows) {
  if (M <= 0) return HIPQ_OK;
  if (K % 256 || lda < K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q8_K: K=%lld must be a multiple of 256 and lda >= K", (long long)K);
  if (((uintptr_t)A & 15) || (lda & 3))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  const int nsb = (int)(K / 256);
  const int64_t total = M * nsb;
  const unsigned grid = (unsigned)((total + 3) / 4);
  hipq::launch_kernel("quantize_q8_K_kernel<Q8K_ROWMMA>", quantize_q8_K_kernel<Q8K_ROWMMA>, dim3(grid), dim3(256), 0, s, A, M, total, nsb, lda,
                     mat_rows, qa->q, qa->d, nullptr, nullptr, (uint16_t *)qa->bsum, nullptr, nullptr);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_quantize_q8_K_tiled(const float *A, int64_t M, int64_t K, int64_t lda, int64_t mat_rows,
                               const QActTiled *qa, hipStream_t s) {
  if (M <= 0) return HIPQ_OK;
  if (K % 256 || lda < K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q8_K: K=%lld must be a multiple of 256 and lda >= K", (long long)K);
  if (((uintptr_t)A & 15) || (lda & 3))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  const int nsb = (int)(K / 256);
  const int64_t units = (int64_t)qa->mtiles * 32 * nsb; /* (row quad, super-block) pairs, padding rows included */
  const unsigned grid = (unsigned)((units + 3) / 4);
  hipq::launch_kernel("quantize_q8_K_tiled_kernel", quantize_q8_K_tiled_kernel, dim3(grid), dim3(256), 0, s, A, M, units, (int)nsb, lda, mat_rows, qa->qt,
                qa->dAt, qa->amin);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq

size_t qact_bytes(int is_k, int64_t M, int64_t K) {
  /* q plane rounded to 256 B, then metadata planes */
  size_t q = ((size_t)M * K + 255) & ~(size_t)255;
  if (is_k) {
    size_t d = ((size_t)M * (K / 256) * 4 + 255) & ~(size_t)255;
    size_t bs = ((size_t)M * (K / 16) * 2 + 255) & ~(size_t)255;
    size_t dg = ((size_t)M * (K / 2) + 255) & ~(size_t)255;
    return q + d + bs + 2 * dg;
  }
  size_t meta = ((size_t)M * (K / 32) * 4 + 255) & ~(size_t)255;
  return q + meta;
}

size_t qact_tiled_bytes(int64_t M, int64_t K) {
  const size_t mpad = (size_t)((M + 127) / 128) * 128, nsb = (size_t)(K / 256);
  return mpad * K + mpad * nsb * 32 + mpad * nsb * 4; /* each a multiple of 256 */
}

QActTiled qact_tiled_carve(void *mem, int64_t M, int64_t K) {
  QActTiled a;
  const size_t mpad = (size_t)((M + 127) / 128) * 128, nsb = (size_t)(K / 256);
  uint8_t *p = (uint8_t *)mem;
  a.M = (int)M;
  a.K = (int)K;
  a.mtiles = (int)(mpad / 128);
  a.qt = (int8_t *)p;
  p += mpad * K;
  a.amin = (uint16_t *)p;
  p += mpad * nsb * 32;
  a.dAt = (float *)p;
  return a;
}

QAct qact_carve(int is_k, void *mem, int64_t M, int64_t K) {
  QAct a;
  uint8_t *p = (uint8_t *)mem;
  a.M = (int)M;
  a.K = (int)K;
  a.q = (int8_t *)p;
  p += ((size_t)M * K + 255) & ~(size_t)255;
  a.meta = nullptr;
  a.d = nullptr;
  a.bsum = nullptr;
  a.ql = nullptr;
  a.qh = nullptr;
  if (is_k) {
    a.d = (float *)p;
    p += ((size_t)M * (K / 256) * 4 + 255) & ~(size_t)255;
    a.bsum = (int16_t *)p;
    p += ((size_t)M * (K / 16) * 2 + 255) & ~(size_t)255;
    a.ql = p;
    p += ((size_t)M * (K / 2) + 255) & ~(size_t)255;
    a.qh = p;
  } else {
    a.meta = (uint32_t *)p;
  }
  return a;
}
