// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm.hip
 * @brief  Prefill GEMM (M > 8) for Q4_0 x Q8_0 on gfx950 int8 matrix cores.
 *         (Q4_K x Q8_K has its own kernel, gemm_q4k.hip.)
 *
 * Replaces the M > 1 branch of __ggml_q4_0_8x8_q8_0_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:330-389 in
 * the reference checkout) and the nntr_gemm_q4_0_8x8_q8_0 kernel behind it
 * (nntr_ggml_impl/nntr_ggml_impl.cpp:650-3259).
 *
 * Structure. A workgroup (4 wavefronts, 2 x 2) owns a 128 x 128 tile of C and
 * walks K in chunks of 256. Per chunk it stages into LDS
 *   - the int8 activations of its 128 rows (32 KB), and
 *   - the int8 expansion of its 128 weight rows: nibbles are unpacked in
 *     registers on the way from HBM to LDS, so HBM only ever carries the packed
 *     4.5-bit form,
 * then every wavefront runs v_mfma_i32_32x32x32_i8 over its 64 x 64 quadrant,
 * one instruction per 32-value block, so each instruction's int32 result is
 * exactly the block's dot product. The per-block scale epilogue runs on the
 * vector ALU: acc += float(dot) * (dw * da).
 * In the MFMA result layout a lane holds one column n and 16 rows m, so the
 * weight-side scales are per-lane registers and the activation-side scales are
 * broadcast reads from LDS.
 *
 * LDS rows are padded to 272 bytes: the 16 lanes of a ds_read_b128 phase then
 * hit 16 disjoint 4-bank groups.
 */
#include "gemv_device.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, KC = 256;
constexpr int LDS_STRIDE = KC + 16; /* bytes per staged row */

struct SmemQ40 {
  int8_t a[BM * LDS_STRIDE];
  int8_t b[BN * LDS_STRIDE];
  float da[8 * BM]; /* [block in chunk][row] */
  float dw[8 * BN]; /* [block in chunk][col] */
};

__device__ __forceinline__ uint32_t nib_to_s8(uint32_t x) {
  /* per byte: (nibble value 0..15) - 8 as int8, no carries between bytes */
  return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

/* Stage the int8 activations of rows [m0, m0+128), chunk kc. */
__device__ __forceinline__ void stage_a(int8_t *sa, const QView &qa, int M, int m0, int kc) {
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int idx = it * 256 + threadIdx.x;
    const int row = idx >> 4, c16 = idx & 15;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (m0 + row < M)
      v = *(const uint4 *)(qa.q + (size_t)(m0 + row) * qa.K + (size_t)kc * KC + c16 * 16);
    *(uint4 *)(sa + row * LDS_STRIDE + c16 * 16) = v;
  }
}

template <int DT>
__device__ __forceinline__ void stage_b(int8_t *sb, const WView &w, int n0, int kc) {
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = it * 256 + threadIdx.x;
    const int row = idx >> 3, c16 = idx & 7;
    uint4 q = make_uint4(0, 0, 0, 0);
    const bool live = n0 + row < w.N;
    if (live)
      q = hipq_ld_stream((const uint4 *)(w.qs + (size_t)(n0 + row) * (w.K >> 1) +
                                         (size_t)kc * (KC / 2) + c16 * 16));
    uint4 lo = make_uint4(q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4);
    uint4 hi = make_uint4((q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                          (q.w >> 4) & HIPQ_M4);
    {
      /* one 32-value block: low nibbles = elements 0..15, high = 16..31 */
      if (live) {
        lo = make_uint4(nib_to_s8(lo.x), nib_to_s8(lo.y), nib_to_s8(lo.z), nib_to_s8(lo.w));
        hi = make_uint4(nib_to_s8(hi.x), nib_to_s8(hi.y), nib_to_s8(hi.z), nib_to_s8(hi.w));
      }
      int8_t *dst = sb + row * LDS_STRIDE + c16 * 32;
      *(uint4 *)dst = lo;
      *(uint4 *)(dst + 16) = hi;
    }
  }
}

/* Row (within the 32 x 32 MFMA tile) of accumulator register r for this lane. */
__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

template <int DT>
__global__ __launch_bounds__(256) void gemm_i8_kernel(WView w, QView qa, int M,
                                                      float *__restrict__ C, int64_t ldc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
  const int l32 = lane & 31, kg = lane >> 5;
  const int nchunks = w.K / KC;

  float accf[2][2][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) accf[i][j][r] = 0.f;

  /* this lane's two weight rows (output columns) */
  int ncol[2];
#pragma unroll
  for (int tn = 0; tn < 2; ++tn) {
    const int n = n0 + wn * 64 + tn * 32 + l32;
    ncol[tn] = n < w.N ? n : w.N - 1;
  }
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  {
    SmemQ40 &sm = *reinterpret_cast<SmemQ40 *>(smem_raw);
    const int nb = w.K >> 5;
    for (int kc = 0; kc < nchunks; ++kc) {
      stage_a(sm.a, qa, M, m0, kc);
      stage_b<HIPQ_Q4_0>(sm.b, w, n0, kc);
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int idx = it * 256 + threadIdx.x;
        const int row = idx >> 3, blk = idx & 7;
        float v = 0.f;
        if (m0 + row < M)
          v = hipq_h2f((uint16_t)(qa.meta[(size_t)(m0 + row) * nb + kc * 8 + blk] & 0xffff));
        sm.da[blk * BM + row] = v;
      }
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int idx = it * 256 + threadIdx.x;
        const int col = idx >> 3, blk = idx & 7;
        float v = 0.f;
        if (n0 + col < w.N) v = hipq_h2f(w.d[(size_t)(n0 + col) * nb + kc * 8 + blk]);
        sm.dw[blk * BN + col] = v;
      }
      __syncthreads();
#pragma unroll 1
      for (int j = 0; j < 8; ++j) {
        v4i a[2], b[2];
        float dw[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          a[t] = *(const v4i *)(sm.a + (wm * 64 + t * 32 + l32) * LDS_STRIDE + j * 32 + kg * 16);
          b[t] = *(const v4i *)(sm.b + (wn * 64 + t * 32 + l32) * LDS_STRIDE + j * 32 + kg * 16);
          dw[t] = sm.dw[j * BN + wn * 64 + t * 32 + l32];
        }
#pragma unroll
        for (int tm = 0; tm < 2; ++tm) {
          float da[16];
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 v =
              *(const float4 *)(sm.da + j * BM + wm * 64 + tm * 32 + 8 * g + 4 * kg);
            da[4 * g] = v.x;
            da[4 * g + 1] = v.y;
            da[4 * g + 2] = v.z;
            da[4 * g + 3] = v.w;
          }
#pragma unroll
          for (int tn = 0; tn < 2; ++tn) {
            const v16i dot = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[tm], b[tn], zero16, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r)
              accf[tm][tn][r] = fmaf((float)dot[r], dw[tn] * da[r], accf[tm][tn][r]);
          }
        }
      }
      __syncthreads();
    }
  }

#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      const int n = n0 + wn * 64 + tn * 32 + l32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + tm * 32 + acc_row(r, lane);
        if (m < M && n < w.N) C[(int64_t)m * ldc + n] = accf[tm][tn][r];
      }
    }
}

} // namespace

namespace hipq {

int launch_gemm(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc,
                hipStream_t s) {
  if (w->K % KC) return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm needs K %% 256 == 0, got %lld", (long long)w->K);
  const dim3 grid((unsigned)((w->N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
  /* the staged tiles need more than the default 64 KB of dynamic LDS */
  static bool lds_opt_in = false;
  if (!lds_opt_in) {
    HIPQ_HIP(hipFuncSetAttribute((const void *)gemm_i8_kernel<HIPQ_Q4_0>,
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(SmemQ40)));
    lds_opt_in = true;
  }
  if (w->dtype == HIPQ_Q4_0) {
    hipLaunchKernelGGL(gemm_i8_kernel<HIPQ_Q4_0>, grid, dim3(256), sizeof(SmemQ40), s, wview(w),
                       qview(*qa), M, C, ldc);
  } else {
    return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm: dtype %d has no MFMA path", w->dtype);
  }
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
