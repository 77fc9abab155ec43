// SPDX-License-Identifier: Apache-2.0
/**
 * @file   ref_shim.cpp
 * @brief  TEST INFRASTRUCTURE ONLY. extern "C" doorway into the reference's own
 *         ggml-interface CPU path, compiled from the reference sources where
 *         they lie (see oracle/Makefile). Nothing here computes anything: every
 *         function forwards to the reference entry point named in its comment.
 *         The resulting library (oracle/_ref/libnntr_ref.so) is used by tests
 *         to pin the C restatement in oracle/nntr_oracle.c and by bench.py's
 *         cpu_baseline leg. It is never linked into the product.
 */
#include <avx2_impl.h>
#include <ggml_interface.h>
#include <nntr_ggml_impl.h>
#include <nntr_ggml_impl_common.h>

#include <cstddef>
#include <cstdint>
#include <omp.h>
#ifdef REF_SHIM_MIXED
#include <bs_thread_pool_manager.hpp>
#endif

extern "C" {

/** nntrainer::__ggml_init, ggml_interface.cpp:24 (fills the fp16 table). */
void ref_init(void) { nntrainer::__ggml_init(); }

/** Half conversions, nntr_ggml_impl_common.h:152-156 (table-backed widen, F16C narrow). */
float ref_fp16_to_fp32(uint16_t h) { return nntr_fp16_to_fp32(h); }
uint16_t ref_fp32_to_fp16(float f) { return nntr_fp32_to_fp16(f); }

/** Weight quantizers, ggml_interface.cpp:26-39. Row = one output column. */
size_t ref_quantize_q4_0(const float *src, void *dst, int64_t nrow,
                         int64_t n_per_row) {
  return nntrainer::__ggml_quantize_q4_0(src, dst, nrow, n_per_row, nullptr);
}
size_t ref_quantize_q4_K(const float *src, void *dst, int64_t nrow,
                         int64_t n_per_row) {
  return nntrainer::__ggml_quantize_q4_K(src, dst, nrow, n_per_row, nullptr);
}
size_t ref_quantize_q6_K(const float *src, void *dst, int64_t nrow,
                         int64_t n_per_row) {
  return nntrainer::__ggml_quantize_q6_K(src, dst, nrow, n_per_row, nullptr);
}

/** Repack to the x8 interleave, ggml_interface.cpp:114-122 (dst first). */
void ref_repack_q4_0_x8(void *dst, void *src, size_t data_size, unsigned N,
                        unsigned K) {
  nntrainer::__ggml_repack_q4_0_to_q4_0_8(dst, src, data_size, N, K);
}
void ref_repack_q4_K_x8(void *dst, void *src, size_t data_size, unsigned N,
                        unsigned K) {
  nntrainer::__ggml_repack_q4_K_to_q4_K_8(dst, src, data_size, N, K);
}

/** Activation quantizers, nntr_ggml_impl.h:70-84. */
void ref_quantize_row_q8_0(const float *x, void *y, int64_t k) {
  nntr_quantize_row_q8_0(x, y, k);
}
void ref_quantize_mat_q8_0_4x8(const float *x, void *y, int64_t k) {
  nntr_quantize_mat_q8_0_4x8(x, y, k);
}
void ref_quantize_row_q8_K(const float *x, void *y, int64_t k) {
  nntr_quantize_row_q8_K(x, y, k);
}
void ref_quantize_mat_q8_K_4x8(const float *x, void *y, int64_t k) {
  nntr_quantize_mat_q8_K_4x8(x, y, k);
}

/** Dequantizers, nntr_ggml_impl.h:86-99. */
void ref_dequantize_row_q4_0(const void *x, float *y, int64_t k) {
  nntr_dequantize_row_q4_0(x, y, k);
}
void ref_dequantize_row_q4_K(const void *x, float *y, int64_t k) {
  nntr_dequantize_row_q4_K(x, y, k);
}
void ref_dequantize_row_q6_K(const void *x, float *y, int64_t k) {
  nntr_dequantize_row_q6_K(x, y, k);
}
void ref_dequantize_row_q8_0(const void *x, float *y, int64_t k) {
  nntr_dequantize_row_q8_0(x, y, k);
}
void ref_dequantize_row_q8_K(const void *x, float *y, int64_t k) {
  nntr_dequantize_row_q8_K(x, y, k);
}

/**
 * The three matmul wrappers the x86 backend dispatches to
 * (x86_compute_backend.cpp:301-341): A fp32 [M x K], B = x8-repacked Q4_0 /
 * Q4_K or canonical Q6_K blocks of W^T [N x K], C fp32 [M x N].
 */
void ref_gemm_q4_0(unsigned M, unsigned N, unsigned K, const float *A,
                   const void *B, float *C) {
  nntrainer::__ggml_q4_0_8x8_q8_0_GEMM(M, N, K, A, K, B, N, C, N);
}
void ref_gemm_q4_K(unsigned M, unsigned N, unsigned K, const float *A,
                   const void *B, float *C) {
  nntrainer::__ggml_q4_K_8x8_q8_K_GEMM(M, N, K, A, K, B, N, C, N);
}
void ref_gemm_q6_K(unsigned M, unsigned N, unsigned K, const float *A,
                   const void *B, float *C) {
  nntrainer::__ggml_gemm_q6_K<float>(M, N, K, A, K, B, N, C, N);
}

/** Raw block kernels, nntr_ggml_impl.h:22-45, 101-103. */
void ref_gemv_q4_0_8x8_q8_0(int n, float *s, size_t bs, const void *vx,
                            const void *vy, int nr, int nc) {
  nntr_gemv_q4_0_8x8_q8_0(n, s, bs, vx, vy, nr, nc);
}
void ref_gemm_q4_0_8x8_q8_0(int n, float *s, size_t bs, const void *vx,
                            const void *vy, int nr, int nc) {
  nntr_gemm_q4_0_8x8_q8_0(n, s, bs, vx, vy, nr, nc);
}
void ref_gemv_q4_K_8x8_q8_K(int n, float *s, size_t bs, const void *vx,
                            const void *vy, int nr, int nc) {
  nntr_gemv_q4_K_8x8_q8_K(n, s, bs, vx, vy, nr, nc);
}
void ref_gemm_q4_K_8x8_q8_K(int n, float *s, size_t bs, const void *vx,
                            const void *vy, int nr, int nc) {
  nntr_gemm_q4_K_8x8_q8_K(n, s, bs, vx, vy, nr, nc);
}
float ref_vec_dot_q6_K_q8_K(unsigned K, const void *vq6, const void *vq8) {
  return nntrainer::__ggml_vec_dot_q6_K_q8_K(K, vq6, vq8);
}

/** nntrainer::swiglu of an x86 build, x86_compute_backend.cpp:286-292 -> avx2_impl.cpp:906-993. */
void ref_swiglu(unsigned n, float *x, const float *y, const float *z) {
  nntrainer::avx2::swiglu(n, x, y, z);
}
void ref_swiglu_alpha(unsigned n, float *x, const float *y, const float *z,
                      float alpha) {
  nntrainer::avx2::swiglu(n, x, y, z, alpha);
}
/** nntrainer::clamp of an x86 build, avx2_impl.cpp:1811-1833. */
void ref_clamp(const float *in, float *out, size_t n, float lo, float hi) {
  nntrainer::avx2::clamp(in, out, n, lo, hi);
}

/** Thread control for the timed baseline. The OpenMP front-end takes its count from
 * OpenMP; the thread-pool front-end sizes its pool itself
 * (bs_thread_pool_manager.hpp:41) and reports it here. */
void ref_set_threads(int n) { omp_set_num_threads(n); }
#ifdef REF_SHIM_MIXED
int ref_max_threads(void) {
  return (int)nntrainer::ThreadPoolManager::Global().getThreadPool().get_thread_count();
}
int ref_front_end_is_thread_pool(void) { return 1; }
#else
int ref_max_threads(void) { return omp_get_max_threads(); }
int ref_front_end_is_thread_pool(void) { return 0; }
#endif
}
