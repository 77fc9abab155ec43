// SPDX-License-Identifier: Apache-2.0
/**
 * @file   bench_kernels.hip
 * @brief  The ceiling kernels of hipq_bench.h: what the int8 matrix instruction
 *         sustains on this device when nothing else is issued, and what a kernel
 *         that does nothing but read device memory gets out of it.
 */
#include "hipq_bench.h"
#include "hipq_internal.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_ceiling_kernel(int iters, int *sink, long long *clocks) {
  const int lane = threadIdx.x & 63;
  v16i d0 = {0}, d1 = {0}, d2 = {0}, d3 = {0};
  const v4i a = {lane, 1, 2, 3}, b = {3, 2, 1, lane};
  const long long c0 = __builtin_readcyclecounter(), r0 = wall_clock64();
  for (int i = 0; i < iters; ++i) {
    d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, d0, 0, 0, 0);
    d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, d1, 0, 0, 0);
    d2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, d2, 0, 0, 0);
    d3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, d3, 0, 0, 0);
  }
  const long long c1 = __builtin_readcyclecounter(), r1 = wall_clock64();
  const int res = d0[0] + d1[1] + d2[2] + d3[3];
  if (res == 0x7fffffff) sink[threadIdx.x] = res; /* keeps the results alive */
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = c1 - c0; /* shader clocks */
    clocks[1] = r1 - r0; /* 100 MHz ticks */
  }
}

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

/* Every wavefront walks its own contiguous share of the buffer in steps of DEPTH KB, DEPTH
 * non-temporal 128-bit loads a lane in flight (each load instruction covers 1 KB of consecutive
 * memory), the way the GEMV kernels stream a weight. */
template <int DEPTH>
__global__ __launch_bounds__(256) void hbm_read_ceiling_kernel(const unsigned char *p, long long kb_per_wave,
                                                               unsigned *sink) {
  const int lane = threadIdx.x & 63;
  const long long wave = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  __amdgpu_buffer_rsrc_t r =
    __builtin_amdgcn_make_buffer_rsrc((void *)(p + wave * kb_per_wave * 1024), 0, (int)(kb_per_wave * 1024), 0x00020000);
  u4 acc = {0, 0, 0, 0};
  /* two halves of DEPTH / 2 loads in turn, the next half asked for before the current one is consumed, so that
   * the wavefront always has loads in flight; past its share's end the loads name the descriptor's end and
   * return zeros without touching memory (unconditional, so that the waits can count them) */
  constexpr int HALF = DEPTH / 2;
  u4 a[HALF], b[HALF];
#pragma unroll
  for (int i = 0; i < HALF; ++i) a[i] = __builtin_amdgcn_raw_buffer_load_b128(r, lane * 16, i * 1024, 2);
  for (long long k = 0; k + DEPTH <= kb_per_wave; k += DEPTH) {
#pragma unroll
    for (int i = 0; i < HALF; ++i)
      b[i] = __builtin_amdgcn_raw_buffer_load_b128(r, lane * 16, (int)(k + HALF + i) * 1024, 2);
#pragma unroll
    for (int i = 0; i < HALF; ++i) acc ^= a[i];
#pragma unroll
    for (int i = 0; i < HALF; ++i)
      a[i] = __builtin_amdgcn_raw_buffer_load_b128(r, lane * 16, (int)(k + DEPTH + i) * 1024, 2);
#pragma unroll
    for (int i = 0; i < HALF; ++i) acc ^= b[i];
  }
  const unsigned x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (x == 0x12345678u) sink[threadIdx.x] = x; /* keeps the loads alive; the buffer holds zeros */
}

} // namespace

extern "C" int hipq_bench_hbm_read_ceiling(int64_t bytes, int regions, int waves_per_simd, void *stream, float *tbs) {
  using hipq::fail;
  if (!tbs || bytes < (int64_t)1 << 20 || bytes > (int64_t)1 << 33 || regions < 1 || regions > 64 ||
      bytes * regions > (int64_t)1 << 35 || waves_per_simd < 1 || waves_per_simd > 8)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad read ceiling arguments");
  hipStream_t s = (hipStream_t)stream;
  int dev = 0, cus = 0;
  HIPQ_HIP(hipGetDevice(&dev));
  HIPQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  constexpr int DEPTH = 8;
  const int wg = cus * waves_per_simd; /* four wavefronts a workgroup: one per SIMD */
  const long long waves = (long long)wg * 4;
  long long kb_per_wave = bytes / 1024 / waves / DEPTH * DEPTH;
  if (kb_per_wave < DEPTH) kb_per_wave = DEPTH;
  if (kb_per_wave * 1024 > 0x7fffffffLL) return fail(HIPQ_ERR_INVALID_ARGUMENT, "a wavefront's share exceeds 2 GiB");
  const size_t total = (size_t)(kb_per_wave * 1024 * waves); /* one region */
  unsigned char *buf = nullptr;
  unsigned *sink = nullptr;
  HIPQ_HIP(hipMalloc((void **)&buf, total * regions));
  hipError_t e = hipMalloc((void **)&sink, 256 * sizeof(unsigned));
  if (e == hipSuccess) e = hipMemsetAsync(buf, 0, total * regions, s);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (e == hipSuccess) e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  /* One region: the first launch warms up and the best of three more counts. Several regions
   * (together larger than the last-level cache): one round over all of them warms up, and the
   * launches of a second round, each on memory last touched a whole round ago, are timed as one
   * run of back-to-back launches. */
  float best = 0.f;
  if (regions == 1) {
    for (int pass = 0; pass < 4 && e == hipSuccess; ++pass) {
      float ms = 0.f;
      e = hipEventRecord(e0, s);
      hipLaunchKernelGGL(hbm_read_ceiling_kernel<DEPTH>, dim3(wg), dim3(256), 0, s, buf, kb_per_wave, sink);
      if (e == hipSuccess) e = hipGetLastError();
      if (e == hipSuccess) e = hipEventRecord(e1, s);
      if (e == hipSuccess) e = hipEventSynchronize(e1);
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
      if (e == hipSuccess && pass > 0 && ms > 0.f) {
        const float r = (float)((double)total / (ms * 1e-3) / 1e12);
        if (r > best) best = r;
      }
    }
  } else {
    for (int round = 0; round < 2 && e == hipSuccess; ++round) {
      float ms = 0.f;
      e = hipEventRecord(e0, s);
      for (int g = 0; g < regions; ++g)
        hipLaunchKernelGGL(hbm_read_ceiling_kernel<DEPTH>, dim3(wg), dim3(256), 0, s, buf + (size_t)g * total,
                           kb_per_wave, sink);
      if (e == hipSuccess) e = hipGetLastError();
      if (e == hipSuccess) e = hipEventRecord(e1, s);
      if (e == hipSuccess) e = hipEventSynchronize(e1);
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
      if (e == hipSuccess && round == 1 && ms > 0.f) best = (float)((double)total * regions / (ms * 1e-3) / 1e12);
    }
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (sink) (void)hipFree(sink);
  (void)hipFree(buf);
  if (e != hipSuccess) return fail(HIPQ_ERR_RUNTIME, "read ceiling kernel: %s", hipGetErrorString(e));
  *tbs = best;
  return HIPQ_OK;
}

extern "C" int hipq_bench_mfma_ceiling(float target_ms, void *stream, float *tops, float *ghz) {
  using hipq::fail;
  if (!tops || !ghz || !(target_ms > 0.f)) return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad ceiling arguments");
  hipStream_t s = (hipStream_t)stream;
  int dev = 0, cus = 0;
  HIPQ_HIP(hipGetDevice(&dev));
  HIPQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  int *sink = nullptr;
  long long *clocks = nullptr;
  HIPQ_HIP(hipMalloc((void **)&sink, 256 * sizeof(int)));
  HIPQ_HIP(hipMalloc((void **)&clocks, 2 * sizeof(long long)));
  hipEvent_t e0, e1;
  HIPQ_HIP(hipEventCreate(&e0));
  HIPQ_HIP(hipEventCreate(&e1));
  const int wg = cus * 3; /* three workgroups of four wavefronts per CU: three per SIMD */
  /* 4 instructions of 32 clocks per iteration and wavefront, three wavefronts per SIMD, ~2.4 GHz */
  int iters = (int)(target_ms * 1e-3 * 2.4e9 / (4 * 32 * 3));
  if (iters < 1000) iters = 1000;
  float ms = 0.f;
  int rc = HIPQ_OK;
  for (int pass = 0; pass < 2 && !rc; ++pass) { /* the first pass warms the clocks up */
    hipError_t e = hipEventRecord(e0, s);
    hipLaunchKernelGGL(mfma_ceiling_kernel, dim3(wg), dim3(256), 0, s, iters, sink, clocks);
    if (e == hipSuccess) e = hipGetLastError();
    if (e == hipSuccess) e = hipEventRecord(e1, s);
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess) rc = fail(HIPQ_ERR_RUNTIME, "ceiling kernel: %s", hipGetErrorString(e));
  }
  long long h[2] = {0, 1};
  if (!rc && hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess)
    rc = fail(HIPQ_ERR_RUNTIME, "ceiling kernel: copy failed");
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(sink);
  (void)hipFree(clocks);
  if (rc) return rc;
  const double ops = 2.0 * 32 * 32 * 32 * 4.0 * (double)iters * 4.0 * wg; /* per instruction x wavefronts */
  *tops = (float)(ops / (ms * 1e-3) / 1e12);
  *ghz = (float)((double)h[0] * 0.1 / (double)h[1]); /* clocks per 10 ns tick */
  return HIPQ_OK;
}
