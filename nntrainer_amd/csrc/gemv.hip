// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemv.hip
 * @brief  Decode GEMV kernels (M = 1, and 2..8 activation rows in one pass over
 *         the weights) for Q4_0, Q4_K and Q6_K weights on gfx950.
 *
 * Replaces the M == 1 branches of __ggml_q4_0_8x8_q8_0_GEMM,
 * __ggml_q4_K_8x8_q8_K_GEMM and __ggml_gemm_q6_K
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:303-329,
 * 404-431, 519-535 in the reference checkout) and the gemv / vec_dot kernels
 * they call; outputs are bit-identical to those kernels (see gemv_device.h).
 *
 * Launch shape: 256 threads = 4 wavefronts per workgroup, each wavefront owns G
 * consecutive output columns (G = 8 for one activation row), so a matrix with N
 * columns launches N / 32 workgroups: 384 for N = 12288, 4748 for the 151936-row
 * lm_head. The kernel is bound by HBM: per output column it reads the column's
 * packed weights exactly once, 16 bytes per lane per load.
 */
#include "gemv_device.h"

namespace {

template <int DT, int T, int R>
__global__ __launch_bounds__(256) void gemv_kernel(WView w, QView qa, int M, int pair_rows,
                                                   float *__restrict__ C, int64_t ldc) {
  constexpr int G = GemvGroup<DT, R>::G;
  extern __shared__ uint32_t gemv_lds[];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = gemv_lds + wave * GemvGroup<DT, R>::LDS_DWORDS;
  const int row0 = (blockIdx.x * 4 + wave) * G;
  int arow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) arow[r] = r < M ? r : M - 1;
  const GemvOut o = gemv_engine<DT, T, R, G>(w, row0, qa, arow, pair_rows, lds);
  if (o.valid && row0 + o.g < w.N && o.r < M) C[(int64_t)o.r * ldc + row0 + o.g] = o.v;
}

template <int DT, int T, int R>
int launch_one(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
               hipStream_t s) {
  constexpr int G = GemvGroup<DT, R>::G;
  const unsigned grid = (unsigned)((w->N + 4 * G - 1) / (4 * G));
  const size_t lds = 4 * GemvGroup<DT, R>::LDS_DWORDS * sizeof(uint32_t);
  hipLaunchKernelGGL((gemv_kernel<DT, T, R>), dim3(grid), dim3(256), lds, s, wview(w), qview(*qa), M,
                     pair_rows, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int R>
int launch_t(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
             hipStream_t s) {
  /* units of work per row: 32-weight units for Q4_0 / Q4_K, 64-weight for Q6_K */
  const int64_t units = (DT == HIPQ_Q6_K) ? w->K / 64 : w->K / 32;
  if (GemvGroup<DT, R>::T16_OK && units < 64)
    return launch_one<DT, (GemvGroup<DT, R>::T16_OK ? 16 : 64), R>(w, qa, M, pair_rows, C, ldc, s);
  return launch_one<DT, 64, R>(w, qa, M, pair_rows, C, ldc, s);
}

template <int DT>
int launch_r(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
             hipStream_t s) {
  if (M == 1) return launch_t<DT, 1>(w, qa, M, pair_rows, C, ldc, s);
  if (M == 2) return launch_t<DT, 2>(w, qa, M, pair_rows, C, ldc, s);
  if (M <= 4) return launch_t<DT, 4>(w, qa, M, pair_rows, C, ldc, s);
  return launch_t<DT, 8>(w, qa, M, pair_rows, C, ldc, s);
}

} // namespace

namespace hipq {

int launch_gemv(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
                hipStream_t s) {
  if (M < 1 || M > 8) return fail(HIPQ_ERR_INVALID_ARGUMENT, "gemv handles 1..8 rows, got %d", M);
  switch (w->dtype) {
  case HIPQ_Q4_0:
    return launch_r<HIPQ_Q4_0>(w, qa, M, pair_rows, C, ldc, s);
  case HIPQ_Q4_K:
    return launch_r<HIPQ_Q4_K>(w, qa, M, pair_rows, C, ldc, s);
  case HIPQ_Q6_K:
    return launch_r<HIPQ_Q6_K>(w, qa, M, pair_rows, C, ldc, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", w->dtype);
}

} // namespace hipq
