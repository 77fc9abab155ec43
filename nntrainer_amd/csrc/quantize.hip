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
#include "hipq_internal.h"

namespace {

constexpr float kRoundMagic = 12582912.f; /* 1.5 * 2^23 */

__device__ __forceinline__ int magic_to_int(float biased) {
  return (int)(__float_as_uint(biased) & 0x007fffffu) - 0x00400000;
}

__device__ __forceinline__ int pack4(int a, int b, int c, int d) {
  return (a & 0xff) | ((b & 0xff) << 8) | ((c & 0xff) << 16) | ((d & 0xff) << 24);
}

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

  float amax = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
  amax = hipq_group_max<8>(amax);

  const float d = __fdiv_rn(amax, 127.f);
  const float id = (amax != 0.0f) ? __fdiv_rn(127.f, amax) : 0.0f;
  const int q0 = (int)rintf(__fmul_rn(x.x, id));
  const int q1 = (int)rintf(__fmul_rn(x.y, id));
  const int q2 = (int)rintf(__fmul_rn(x.z, id));
  const int q3 = (int)rintf(__fmul_rn(x.w, id));
  const int packed = pack4(q0, q1, q2, q3);
  const uint16_t dh = hipq_f2h(d);

  if (CANONICAL) {
    if (!live) return;
    uint8_t *o = canon_out + blk * 34;
    if (sub == 0) *(uint16_t *)o = dh;
    uint16_t *qs = (uint16_t *)(o + 2 + sub * 4);
    qs[0] = (uint16_t)(packed & 0xffff);
    qs[1] = (uint16_t)((unsigned)packed >> 16);
  } else {
    int bsum = hipq_group_sum_i<8>(q0 + q1 + q2 + q3);
    if (!live) return;
    *(int *)(q_out + (m * nb + b) * 32 + sub * 4) = packed;
    if (sub == 0) meta_out[m * nb + b] = (uint32_t)dh | ((uint32_t)(bsum & 0xffff) << 16);
  }
}

/* ---- Q8_K ---------------------------------------------------------------- */
enum { Q8K_PLANES = 0, Q8K_CANONICAL = 1, Q8K_TILED = 2, Q8K_ROWMMA = 3 };

/* One wavefront per (row, super-block). In the tiled mode the grid also covers
 * the padding rows M .. n_sb_total / nsb - 1, which are written as zeros. */
template <int MODE>
__global__ __launch_bounds__(256) void quantize_q8_K_kernel(
  const float *__restrict__ A, int64_t M, int64_t n_sb_total, int nsb, int64_t lda,
  int64_t mat_rows, int8_t *__restrict__ q_out, float *__restrict__ d_out,
  int16_t *__restrict__ bsum_out, uint8_t *__restrict__ canon_out,
  uint16_t *__restrict__ amin_out, uint16_t *__restrict__ ql_out, uint16_t *__restrict__ qh_out) {
  const int lane = threadIdx.x & 63;
  int64_t sb = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const bool live = sb < n_sb_total; /* uniform per wavefront */
  if (!live) return;
  const int64_t m = sb / nsb;
  const int b = (int)(sb - m * nsb);
  float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (m < M) xv = *(const float4 *)(A + m * lda + (int64_t)b * 256 + lane * 4);
  const float x[4] = {xv.x, xv.y, xv.z, xv.w};

  float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
  amax = hipq_group_max<64>(amax);

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
    const float vmax = __shfl(cand, first, HIPQ_WAVE);
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
  } else if (MODE == Q8K_TILED) {
    const int64_t mt = m >> 7;
    const int r = (int)(m & 127);
    /* lane holds elements 4*lane .. 4*lane+3 of the super-block: sub-block lane / 8,
     * whose 16-value half (lane / 4) % 2 is one 16-byte operand. The GEMM's lane
     * (row, g) takes sub-blocks 4g .. 4g+3, two 32-deep steps each, so the operand
     * belongs to step s = 2 * (sub-block % 4) + half of lane group g = sub-block / 4;
     * within the operand the 8 even values come first, then the 8 odd ones (the
     * order in which the weights' nibble bytes unpack). */
    const int jb = lane >> 3, g = jb >> 2;
    const int st = 2 * (jb & 3) + ((lane >> 2) & 1);
    const int64_t tile = (mt * (2 * nsb) + b * 2 + (st >> 2)) * 16384;
    const int off = ((r >> 5) * 4 + (st & 3)) * 1024 + (g * 32 + (r & 31)) * 16 + (lane & 3) * 2;
    *(uint16_t *)(q_out + tile + off) = (uint16_t)((q[0] & 0xff) | ((q[2] & 0xff) << 8));
    *(uint16_t *)(q_out + tile + off + 8) = (uint16_t)((q[1] & 0xff) | ((q[3] & 0xff) << 8));
    const int64_t rb = (mt * nsb + b) * 128 + r;
    if (lane == 0) d_out[rb] = d;
    const int bs = gsum + __shfl_xor(gsum, 4, HIPQ_WAVE); /* two 16-value groups = one sub-block */
    if ((lane & 7) == 0) {
      const int l6 = bs & 63;
      amin_out[rb * 16 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)l6));
      amin_out[rb * 16 + 8 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)(bs - l6)));
    }
  } else if (MODE == Q8K_ROWMMA) {
    /* row-major, each 16-value group stored as its 8 even then its 8 odd values:
     * this lane's four values are elements 4l .. 4l+3 of group lane / 4 */
    int8_t *o = q_out + sb * 256 + (lane >> 2) * 16 + (lane & 3) * 2;
    *(uint16_t *)o = (uint16_t)((q[0] & 0xff) | ((q[2] & 0xff) << 8));
    *(uint16_t *)(o + 8) = (uint16_t)((q[1] & 0xff) | ((q[3] & 0xff) << 8));
    if (lane == 0) d_out[sb] = d;
    const int bs = gsum + __shfl_xor(gsum, 4, HIPQ_WAVE); /* two 16-value groups = one sub-block */
    if ((lane & 7) == 0) {
      const int l6 = bs & 63;
      amin_out[sb * 16 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)l6));
      amin_out[sb * 16 + 8 + (lane >> 3)] = __half_as_ushort(__float2half_rn((float)(bs - l6)));
    }
  } else {
    *(int *)(q_out + sb * 256 + lane * 4) = packed;
    if (lane == 0) d_out[sb] = d;
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
  hipLaunchKernelGGL(quantize_q8_K_kernel<Q8K_TILED>, dim3(grid), dim3(256), 0, s, A, M, total, nsb, lda,
                     mat_rows, qa->qt, qa->dAt, nullptr, nullptr, qa->amin, nullptr, nullptr);
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
