// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemv.hip
 * @brief  Decode GEMV kernels (M = 1, and 2..8 activation rows in one pass over
 *         the weights) for Q4_0, Q4_K and Q6_K weights on gfx950.
 *
 * Replaces the M == 1 branches of __ggml_q4_0_8x8_q8_0_GEMM,
 * __ggml_q4_K_8x8_q8_K_GEMM and __ggml_gemm_q6_K
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:303-329,
 * 404-431, 519-535 in the reference checkout) and the gemv kernels they call.
 *
 * Launch shape: 256 threads = 4 wavefronts per workgroup; a group of T lanes
 * owns one output column, so a workgroup produces 4 * 64 / T columns and a
 * matrix with N columns launches N * T / 256 workgroups -- thousands for the
 * decode shapes, far more than the 256 compute units. The kernel is bound by
 * HBM: per output column it reads the column's packed weights exactly once.
 */
#include "gemv_device.h"

namespace {

template <int DT, int T, int R>
__global__ __launch_bounds__(256) void gemv_kernel(WView w, QView qa, int M, float *__restrict__ C,
                                                   int64_t ldc) {
  constexpr int ROWS_PER_WAVE = 64 / T;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int tl = lane % T;
  int row = (blockIdx.x * 4 + wave) * ROWS_PER_WAVE + lane / T;
  const bool live = row < w.N;
  if (!live) row = w.N - 1; /* stay in the reductions, store nothing */
  int arow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) arow[r] = r < M ? r : M - 1;
  float out[R];
  gemv_rows<DT, T, R>(w, row, tl, qa, arow, out);
  if (live && tl == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < M) C[(int64_t)r * ldc + row] = out[r];
  }
}

template <int DT, int T, int R>
int launch_one(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  constexpr int ROWS_PER_BLOCK = 4 * (64 / T);
  const unsigned grid = (unsigned)((w->N + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
  hipLaunchKernelGGL((gemv_kernel<DT, T, R>), dim3(grid), dim3(256), 0, s, wview(w), qview(*qa), M,
                     C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int T>
int launch_r(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  if (M == 1) return launch_one<DT, T, 1>(w, qa, M, C, ldc, s);
  if (M == 2) return launch_one<DT, T, 2>(w, qa, M, C, ldc, s);
  if (M <= 4) return launch_one<DT, T, 4>(w, qa, M, C, ldc, s);
  return launch_one<DT, T, 8>(w, qa, M, C, ldc, s);
}

template <int DT>
int launch_t(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  /* units of work per row: 32-weight units for Q4_0 / Q4_K, 64-weight for Q6_K */
  const int64_t units = (DT == HIPQ_Q6_K) ? w->K / 64 : w->K / 32;
  if (units >= 64) return launch_r<DT, 64>(w, qa, M, C, ldc, s);
  return launch_r<DT, 16>(w, qa, M, C, ldc, s);
}

} // namespace

namespace hipq {

int launch_gemv(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc,
                hipStream_t s) {
  if (M < 1 || M > 8) return fail(HIPQ_ERR_INVALID_ARGUMENT, "gemv handles 1..8 rows, got %d", M);
  switch (w->dtype) {
  case HIPQ_Q4_0:
    return launch_t<HIPQ_Q4_0>(w, qa, M, C, ldc, s);
  case HIPQ_Q4_K:
    return launch_t<HIPQ_Q4_K>(w, qa, M, C, ldc, s);
  case HIPQ_Q6_K:
    return launch_t<HIPQ_Q6_K>(w, qa, M, C, ldc, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", w->dtype);
}

} // namespace hipq
