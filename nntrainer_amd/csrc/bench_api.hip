// SPDX-License-Identifier: Apache-2.0
/**
 * @file   bench_api.hip
 * @brief  Measurement and test helpers of libhipq_bench.so (hipq_bench.h). This library is not
 *         the product: it links libhipq.so and reaches it through the public C ABI only (the
 *         timed loop is a loop of hipq_matmul calls), plus its own copy of the activation
 *         quantizer's object code for the test that looks at an internal buffer layout.
 */
#include <cstdarg>
#include <cstdio>

#include "hipq_bench.h"
#include "hipq_internal.h"

namespace {
thread_local char bench_error[512] = "";
}

namespace hipq {
/* what the quantizer's object code expects from the library it is linked into */
thread_local LaunchLog launch_log;
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(bench_error, sizeof(bench_error), fmt, ap);
  va_end(ap);
  return code;
}
} // namespace hipq

extern "C" {

const char *hipq_bench_last_error(void) { return bench_error; }

int hipq_bench_matmul_loop(int n_weights, const hipq_weight_t *w, const float *A, int64_t M, int64_t lda, float *C,
                           int64_t ldc, int iters, void *stream, float *ms_per_call) {
  if (n_weights <= 0 || !w || iters <= 0 || !ms_per_call)
    return hipq::fail(HIPQ_ERR_INVALID_ARGUMENT, "bad timing arguments");
  hipStream_t s = (hipStream_t)stream;
  /* one untimed call per weight first: workspace and tile copies exist before the events */
  for (int i = 0; i < n_weights; ++i) {
    const int rc = hipq_matmul(w[i], A, M, lda, C, ldc, HIPQ_MEM_DEVICE, stream);
    if (rc) return hipq::fail(rc, "hipq_matmul: %s", hipq_last_error());
  }
  hipEvent_t e0, e1;
  HIPQ_HIP(hipEventCreate(&e0));
  HIPQ_HIP(hipEventCreate(&e1));
  HIPQ_HIP(hipStreamSynchronize(s));
  HIPQ_HIP(hipEventRecord(e0, s));
  int rc = HIPQ_OK;
  for (int it = 0; it < iters && !rc; ++it) rc = hipq_matmul(w[it % n_weights], A, M, lda, C, ldc, HIPQ_MEM_DEVICE, stream);
  hipError_t er = hipEventRecord(e1, s);
  if (er == hipSuccess) er = hipEventSynchronize(e1);
  float ms = 0.f;
  if (er == hipSuccess) er = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc) return hipq::fail(rc, "hipq_matmul: %s", hipq_last_error());
  if (er != hipSuccess) return hipq::fail(HIPQ_ERR_RUNTIME, "timing: %s", hipGetErrorString(er));
  *ms_per_call = ms / (float)iters;
  return HIPQ_OK;
}

int64_t hipq_bench_tiled_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % 256) return HIPQ_ERR_INVALID_ARGUMENT;
  return (int64_t)::qact_tiled_bytes(M, K);
}

int hipq_bench_quantize_tiled(const float *A, int64_t M, int64_t K, int64_t lda, void *out, void *stream) {
  if (!A || !out || M <= 0 || K <= 0) return hipq::fail(HIPQ_ERR_INVALID_ARGUMENT, "bad argument");
  const QActTiled qa = ::qact_tiled_carve(out, M, K);
  return hipq::launch_quantize_q8_K_tiled(A, M, K, lda, (M / 4) * 4, &qa, (hipStream_t)stream);
}

} /* extern "C" */
