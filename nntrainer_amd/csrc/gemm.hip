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
 * Structure. A workgroup (4 wavefronts, 2 x 2) owns a 64 x 64 tile of C, each
 * wavefront 32 x 32, and walks K in chunks of 256. Q4_0 has one fp16 scale per 32
 * weights and Q8_0 one per 32 activations, so every v_mfma_i32_32x32x32_i8 is one
 * block whose exact int32 sums are scaled on the vector ALU:
 * acc += float(dot) * (dw * da), three instructions per sum, which bounds this
 * formulation well below the matrix peak (48 vector instructions per MFMA). What
 * the kernel therefore optimises is occupancy and latency: the tile is small so
 * that the FC shapes of a small decoder (N = 1024 .. 3072, 512 rows) still give
 * hundreds of workgroups, four of them fit a CU (38 KB of LDS each), and the next
 * chunk's global loads are in flight in registers while the current one is
 * computed. Per chunk a workgroup stages into LDS
 *   - the int8 activations of its 64 rows (16 KB), and
 *   - the int8 expansion of its 64 weight rows: nibbles are unpacked in registers
 *     on the way from HBM to LDS, so HBM only ever carries the packed 4.5-bit form,
 *   - the scales of both sides, [block][row] and [block][column].
 * In the MFMA result layout a lane holds one column n and 16 rows m, so the
 * weight-side scale is a per-lane value and the activation-side scales are
 * 128-bit LDS reads.
 *
 * LDS rows are padded to 272 bytes: the 16 lanes of a ds_read_b128 phase then
 * hit 16 disjoint 4-bank groups.
 */
#include "gemv_device.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 64, BN = 64, KC = 256;
constexpr int LDS_STRIDE = KC + 16; /* bytes per staged row */

struct SmemQ40 {
  int8_t a[BM * LDS_STRIDE];
  int8_t b[BN * LDS_STRIDE];
  float da[8 * BM]; /* [block in chunk][row] */
  float dw[8 * BN]; /* [block in chunk][col] */
};
static_assert(sizeof(SmemQ40) * 4 <= 160 * 1024, "four workgroups per CU");

__device__ __forceinline__ uint32_t nib_to_s8(uint32_t x) {
  /* per byte: (nibble value 0..15) - 8 as int8, no carries between bytes */
  return ((x | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
}

/* One chunk of a workgroup's inputs, as loaded (registers of one thread). */
struct Chunk {
  v4i a[4];      /* activations: piece idx = it * 256 + t -> row idx / 16, 16-byte column idx % 16 */
  v4i b[2];      /* nibbles: piece idx = it * 256 + t -> row idx / 8, block idx % 8 */
  uint32_t ma[2]; /* activation block metadata (fp16 d in the low half): row idx / 8, block idx % 8 */
  uint16_t dw[2]; /* weight scales, same indexing */
};

__device__ __forceinline__ void load_chunk(Chunk &c, const WView &w, const QView &qa, int M, int m0,
                                           int n0, int kc) {
  const int t = threadIdx.x;
  const int nb = w.K >> 5;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = it * 256 + t;
    const int row = min(m0 + (idx >> 4), M - 1); /* rows past M are never stored */
    c.a[it] = *(const v4i *)(qa.q + (size_t)row * qa.K + (size_t)kc * KC + (idx & 15) * 16);
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * 256 + t;
    const int col = min(n0 + (idx >> 3), (int)w.N - 1);
    const int blk = kc * 8 + (idx & 7);
    const uint4 q = hipq_ld_stream((const uint4 *)(w.qs + (size_t)col * (w.K >> 1)) + blk);
    c.b[it] = v4i{(int)q.x, (int)q.y, (int)q.z, (int)q.w};
    c.dw[it] = hipq_ld_global(w.d + (size_t)col * nb + blk);
    const int row = min(m0 + (idx >> 3), M - 1);
    c.ma[it] = qa.meta[(size_t)row * nb + blk];
  }
}

__device__ __forceinline__ void store_chunk(const Chunk &c, SmemQ40 &sm) {
  const int t = threadIdx.x;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = it * 256 + t;
    *(v4i *)(sm.a + (idx >> 4) * LDS_STRIDE + (idx & 15) * 16) = c.a[it];
  }
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * 256 + t;
    const int row = idx >> 3, blk = idx & 7;
    /* one 32-value block: low nibbles = elements 0..15, high = 16..31 */
    v4i lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t x = (uint32_t)c.b[it][e];
      lo[e] = (int)nib_to_s8(x & HIPQ_M4);
      hi[e] = (int)nib_to_s8((x >> 4) & HIPQ_M4);
    }
    int8_t *dst = sm.b + row * LDS_STRIDE + blk * 32;
    *(v4i *)dst = lo;
    *(v4i *)(dst + 16) = hi;
    sm.dw[blk * BN + row] = hipq_h2f(c.dw[it]);
    sm.da[blk * BM + row] = hipq_h2f((uint16_t)(c.ma[it] & 0xffff));
  }
}

/* Row (within the 32 x 32 MFMA tile) of accumulator register r for this lane. */
__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

__global__ __launch_bounds__(256, 4) void gemm_q40_kernel(WView w, QView qa, int M,
                                                          float *__restrict__ C, int64_t ldc) {
  __shared__ SmemQ40 sm;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
  const int l32 = lane & 31, kg = lane >> 5;
  const int nchunks = w.K / KC;
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  float acc[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;

  Chunk c;
  load_chunk(c, w, qa, M, m0, n0, 0);
  const int8_t *pa = sm.a + (wm * 32 + l32) * LDS_STRIDE + kg * 16;
  const int8_t *pb = sm.b + (wn * 32 + l32) * LDS_STRIDE + kg * 16;
  for (int kc = 0; kc < nchunks; ++kc) {
    store_chunk(c, sm);
    __syncthreads();
    if (kc + 1 < nchunks) load_chunk(c, w, qa, M, m0, n0, kc + 1); /* in flight during the chunk */
#pragma unroll 2
    for (int j = 0; j < 8; ++j) {
      const v4i a = *(const v4i *)(pa + j * 32);
      const v4i b = *(const v4i *)(pb + j * 32);
      const float dw = sm.dw[j * BN + wn * 32 + l32];
      const v16i dot = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero16, 0, 0, 0);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 da = *(const float4 *)(sm.da + j * BM + wm * 32 + 8 * g + 4 * kg);
        acc[4 * g] = fmaf((float)dot[4 * g], dw * da.x, acc[4 * g]);
        acc[4 * g + 1] = fmaf((float)dot[4 * g + 1], dw * da.y, acc[4 * g + 1]);
        acc[4 * g + 2] = fmaf((float)dot[4 * g + 2], dw * da.z, acc[4 * g + 2]);
        acc[4 * g + 3] = fmaf((float)dot[4 * g + 3], dw * da.w, acc[4 * g + 3]);
      }
    }
    __syncthreads();
  }

  const int n = n0 + wn * 32 + l32;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + wm * 32 + acc_row(r, lane);
    if (m < M && n < w.N) C[(int64_t)m * ldc + n] = acc[r];
  }
}

} // namespace

namespace hipq {

int launch_gemm(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc,
                hipStream_t s) {
  if (w->K % KC) return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm needs K %% 256 == 0, got %lld", (long long)w->K);
  if (w->dtype != HIPQ_Q4_0) return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm: dtype %d has no MFMA path here", w->dtype);
  const dim3 grid((unsigned)((w->N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
  hipLaunchKernelGGL(gemm_q40_kernel, grid, dim3(256), 0, s, wview(w), qview(*qa), M, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
