/* SPDX-License-Identifier: Apache-2.0 */
/**
 * @file   hipq_bench.h
 * @brief  Measurement and test helpers exported by libhipq.so for bench.py and the GPU
 *         tests only. They are not part of the product's C ABI (include/hipq.h) and
 *         replace nothing in the reference: event-timed launch loops, a matrix-core
 *         and a memory-read ceiling kernel, and a view of an internal buffer layout for
 *         its parity test.
 */
#ifndef HIPQ_BENCH_H
#define HIPQ_BENCH_H

#include "hipq.h"

#ifdef __cplusplus
extern "C" {
#endif

/** Runs the matmul `iters` times on device buffers, rotating over `n_weights` handles
 *  (distinct copies defeat the last-level cache), brackets the launches with HIP events
 *  recorded on `stream` and returns the average milliseconds per call.
 *  phase 0: whole call (activation quantizer + block-dot kernel);
 *  phase 1: block-dot kernel only, on activations quantized once beforehand;
 *  phase 2: activation quantizer only. */
HIPQ_API int hipq_time_matmul(int n_weights, const hipq_weight_t *w, const float *A, int64_t M,
                              int64_t lda, float *C, int64_t ldc, int iters, int phase, void *stream,
                              float *ms_per_call);

/** `steps` whole matmuls (activation quantizer, then block-dot kernel) as hipq_matmul
 *  enqueues them on `stream`. total_ms: between one event recorded before the first
 *  quantizer and one behind the last product (nothing else is put into the stream, so the
 *  kernels follow each other as they do in a caller's loop). quantizer_ms, product_ms: sums
 *  of the kernels' own durations, taken from a start and a stop event attached to each of
 *  the same launches (hipExtLaunchKernelGGL): what a kernel trace reports for them.
 *  total >= quantizer + product; the difference is the time between the kernels. */
HIPQ_API int hipq_bench_matmul_steps(int n_weights, const hipq_weight_t *w, const float *A, int64_t M,
                                     int64_t lda, float *C, int64_t ldc, int steps, void *stream,
                                     float *total_ms, float *quantizer_ms, float *product_ms);

/** Nothing but v_mfma_i32_32x32x32_i8 on every SIMD of the device (three wavefronts each,
 *  four independent accumulators) for about `target_ms`: the int8 rate the matrix cores
 *  sustain here, in TOP/s, and the shader clock during the run in GHz. */
HIPQ_API int hipq_bench_mfma_ceiling(float target_ms, void *stream, float *tops, float *ghz);

/** A kernel that does nothing but read `bytes` of device memory (allocated, zeroed and freed
 *  by this call; 1 GiB is four times the last-level cache) with `waves_per_simd` wavefronts on
 *  every SIMD, each streaming its own contiguous share with eight non-temporal 128-bit loads a
 *  lane in flight: the read rate in TB/s that the memory system gives a kernel of the GEMV
 *  kernels' access pattern. regions == 1: best of three launches. regions > 1: that many
 *  buffers of `bytes` each, read one per launch in a run of back-to-back launches, every
 *  buffer last touched a whole round earlier (a small weight read cold, launch included). */
HIPQ_API int hipq_bench_hbm_read_ceiling(int64_t bytes, int regions, int waves_per_simd, void *stream, float *tbs);

/** The Q8_K activation quantizer in the form the Q4_K prefill product reads (rows tiled by
 *  128, 16-byte matrix operands; csrc/hipq_internal.h, QActTiled), written into ONE device
 *  buffer `out` of hipq_bench_tiled_bytes(M, K) bytes: the int8 tiles, then the fp16 parts of
 *  the sub-block sums, then the scales. For the test that compares it, value by value, with
 *  the canonical blocks of hipq_quantize_q8_K. A, out: device memory. */
HIPQ_API int64_t hipq_bench_tiled_bytes(int64_t M, int64_t K);
HIPQ_API int hipq_bench_quantize_tiled(const float *A, int64_t M, int64_t K, int64_t lda, void *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPQ_BENCH_H */
