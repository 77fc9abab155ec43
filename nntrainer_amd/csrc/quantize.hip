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

/* One wavefront per (row, super-block). In the tiled mode the grid also covers
 * the padding rows M .. n_sb_total / nsb - 1, which are written as zeros. */
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
    hipLaunchKernelGGL(quantize_q8_0_kernel<true>, dim3(grid), dim3(256), 0, s, A, total, nb, lda,
                       nullptr, nullptr, (uint8_t *)canonical_out);
  else
    hipLaunchKernelGGL(quantize_q8_0_kernel<false>, dim3(grid), dim3(256), 0, s, A, total, nb, lda,
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
    hipLaunchKernelGGL(quantize_q8_K_kernel<Q8K_CANONICAL>, dim3(grid), dim3(256), 0, s, A, M, total,
                       nsb, lda, mat_rows, nullptr, nullptr, nullptr, (uint8_t *)canonical_out, nullptr, nullptr,
                       nullptr);
  else
    hipLaunchKernelGGL(quantize_q8_K_kernel<Q8K_PLANES>, dim3(grid), dim3(256), 0, s, A, M, total, nsb,
                       lda, mat_rows, qa->q, qa->d, qa->bsum, nullptr, nullptr, (uint16_t *)qa->ql,
                       (uint16_t *)qa->qh);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_quantize_q8_K_rowmma(const float *A, int64_t M, int64_t K, int64_t lda, const QAct *qa,
                                hipStream_t s) {
  if (M <= 0) return HIPQ_OK;
  if (K % 256 || lda < K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q8_K: K=%lld must be a multiple of 256 and lda >= K", (long long)K);
  if (((uintptr_t)A & 15) || (lda & 3))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  const int nsb = (int)(K / 256);
  const int64_t total = M * nsb;
  const unsigned grid = (unsigned)((total + 3) / 4);
  hipLaunchKernelGGL(quantize_q8_K_kernel<Q8K_ROWMMA>, dim3(grid), dim3(256), 0, s, A, M, total, nsb, lda,
                     (int64_t)0, qa->q, qa->d, nullptr, nullptr, (uint16_t *)qa->bsum, nullptr, nullptr);
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
  const int64_t total = (int64_t)qa->mtiles * 128 * nsb;
  const unsigned grid = (unsigned)((total + 3) / 4);
  launch_kernel(quantize_q8_K_kernel<Q8K_TILED>, dim3(grid), dim3(256), 0, s, A, M, total, (int)nsb, lda, mat_rows,
                qa->qt, qa->dAt, (int16_t *)nullptr, (uint8_t *)nullptr, qa->amin, (uint16_t *)nullptr,
                (uint16_t *)nullptr);
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
