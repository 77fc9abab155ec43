/* SPDX-License-Identifier: Apache-2.0 */
/**
 * @file   hipq_bench.h
 * @brief  Measurement and test helpers of libhipq_bench.so, a library of its own beside
 *         libhipq.so, for bench.py and the GPU tests only. They are not part of the
 *         product's C ABI (include/hipq.h) and replace nothing in the reference: an
 *         event-timed loop of hipq_matmul calls, a matrix-core and a memory-read ceiling
 *         kernel, and a view of an internal buffer layout for its parity test.
 */
#ifndef HIPQ_BENCH_H
#define HIPQ_BENCH_H

#include "hipq.h"

#ifdef __cplusplus
extern "C" {
#endif

/** `iters` calls of hipq_matmul on device buffers, rotating over `n_weights` handles (distinct
 *  copies defeat the last-level cache), after one untimed call per weight; two HIP events recorded
 *  on `stream` before the first and behind the last call; returns the average milliseconds per
 *  call. Nothing else is put into the stream, so the kernels follow each other as they do in a
 *  caller's loop. The kernels' own durations come from hipq_launch_timing_begin / _end
 *  (include/hipq.h) around such a loop. */
HIPQ_API int hipq_bench_matmul_loop(int n_weights, const hipq_weight_t *w, const float *A, int64_t M,
                                    int64_t lda, float *C, int64_t ldc, int iters, void *stream,
                                    float *ms_per_call);
HIPQ_API const char *hipq_bench_last_error(void);

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
