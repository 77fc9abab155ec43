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
 * consecutive output columns; G = 4 from N = 8192 up (9497 workgroups for the
 * 151936-row lm_head, 768 for N = 12288), 2 or 1 for smaller matrices so that
 * they still fill the 1024 SIMDs. The kernel is bound by
 * HBM: per output column it reads the column's packed weights exactly once,
 * 16 bytes per lane per load, all loads of a group in flight together.
 */
#include <string>
#include <type_traits>

#include "gemv_device.h"
#include "quantize_device.h"

namespace {

template <int DT, int T, int R, int G, bool PW, int FK>
__global__ __launch_bounds__(256) void gemv_kernel(WView w, QView qa, int M, int pair_rows,
                                                   float *__restrict__ C, int64_t ldc) {
  extern __shared__ uint32_t gemv_lds[];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = gemv_lds + wave * GemvLds<DT, R, G, PW>::DWORDS;
  const int row0 = (blockIdx.x * 4 + wave) * G;
  int arow[R];
#pragma unroll
  for (int r = 0; r < R; ++r) arow[r] = r < M ? r : M - 1;
  const GemvOut o = gemv_engine<DT, T, R, G, PW, HIPQ_KCHUNK, FK>(w, row0, qa, arow, pair_rows, lds);
  if (o.valid && row0 + o.g < w.N && o.r < M) C[(int64_t)o.r * ldc + row0 + o.g] = o.v;
}

/* Decode GEMV for large matrices: a wavefront owns GPW consecutive groups of G
 * rows. The activation row is loaded once, and the weight loads of the next
 * group are in flight while the current one is computed, so the HBM stream of a
 * wavefront never drains. T lanes a row (64, or 16 for rows of fewer than 64 units). One chunk only
 * (K <= 4096). */
template <int DT, int T, int G, int GPW, int FK>
__global__ __launch_bounds__(256) void gemv_stream_kernel(WView w, QView qa,
                                                          float *__restrict__ C) {
  typedef GemvCore<DT, T, 1, G, false> E;
  extern __shared__ uint32_t gemv_lds[];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = gemv_lds + wave * GemvLds<DT, 1, G, false>::DWORDS;
  const int first = (blockIdx.x * 4 + wave) * GPW * G;
  if (first >= w.N) return; /* uniform per wavefront; all syncs below are wavefront-local */
  /* FK: the row length where the launcher has seen one of the usual ones (0: any). With it a constant, and the
   * next group's loads issued whether or not the matrix still has those rows (a row past the end is read as
   * the last one), no load sits behind a condition and the waits of a group's arithmetic leave the next
   * group's loads in flight; behind a condition they were waited for with everything else. */
  const int K = FK ? FK : w.K;
  const int arow[1] = {0};
  typename E::Wts W[2];
  typename E::Act A;
  /* the activations' loads first and nothing moved across: a load that the arithmetic needs and that is
   * issued behind the weights' has to wait for all of them */
  E::load_act(A, qa, arow, 0, K);
  __builtin_amdgcn_sched_barrier(0);
  E::load_w(W[0], w, first, 0, K);
#pragma unroll
  for (int i = 0; i < GPW; ++i) {
    const int row0 = first + i * G;
    if (row0 >= w.N) break; /* uniform */
    if (i + 1 < GPW) E::load_w(W[(i + 1) & 1], w, row0 + G, 0, K);
    __builtin_amdgcn_sched_barrier(0);
    typename E::Chain c = E::begin(arow, 0);
    E::compute(W[i & 1], A, K, lds);
    hipq_wave_lds_sync();
    E::chain(c, K, lds);
    hipq_wave_lds_sync();
    const GemvOut o = E::finish(c);
    if (o.valid && row0 + o.g < w.N) C[row0 + o.g] = o.v;
  }
}

/* Decode GEMV on the fp32 activation row itself: the workgroup quantizes the row
 * into LDS (the arithmetic of the quantizer kernels, so the blocks are the same
 * bits) while its weight loads are in flight, and the engine reads the activations
 * from there. Saves the quantizer's launch, which costs more than the redundant
 * quantization as long as the matrix is small. One chunk only (K <= 4096). */
template <int DT> __host__ __device__ constexpr int fused_act_bytes(int K) {
  /* Q8_0: q [K], meta [K/32] u32; Q8_K: q [K], ql [K/2], qh [K/2], bsum [K/16] i16, d [K/256] f32 */
  return ((DT == HIPQ_Q4_0 ? K + K / 8 : 2 * K + K / 8 + K / 64) + 15) & ~15;
}

template <int DT, int T, int G, int NW, int LATE, int FK, int WV = 4, typename Store>
__device__ __forceinline__ void gemv_fused_rows(const WView (&wv)[NW], const float *__restrict__ x, int block,
                                                Store store) {
  static_assert(WV == 4 || (DT != HIPQ_Q4_0 && WV == 12), "wavefronts a workgroup");
  constexpr int XP = 16 / WV + (16 % WV != 0); /* super-blocks of the row a wavefront quantizes, at most (K <= 4096) */
  typedef GemvCore<DT, T, 1, G, false> E;
  const WView &w = wv[0];
  extern __shared__ __attribute__((aligned(16))) uint32_t gemv_lds[];
  /* FK: the row length the launcher has seen, where it is one of the usual ones (0: any). With the length a
   * constant every load of the row and of the weights is issued unconditionally, and the waits can count them:
   * a load behind a condition makes every wait in front of it a wait for nearly all loads in flight. */
  const int K = FK ? FK : w.K;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint8_t *ap = (uint8_t *)gemv_lds;
  uint32_t *lds = gemv_lds + fused_act_bytes<DT>(K) / 4 + wave * GemvLds<DT, 1, G, false>::DWORDS;
  const int row0 = (block * WV + wave) * G;
  const int arow[1] = {0};

  /* the row first (it comes from the cache), then the weights: the wait for the row
   * leaves the weight loads in flight. Positions beyond the row re-read its end. */
  float4 xs[4];
  if (DT == HIPQ_Q4_0) {
    const int nb = K >> 5;
#pragma unroll
    for (int p = 0; p < 4; ++p)
      xs[p] = *(const float4 *)(x + min((int)(threadIdx.x >> 3) + 32 * p, nb - 1) * 32 + (threadIdx.x & 7) * 4);
  } else {
    const int nsb = K >> 8;
#pragma unroll
    for (int p = 0; p < XP; ++p) xs[p] = *(const float4 *)(x + min(wave + WV * p, nsb - 1) * 256 + lane * 4);
  }
  /* LATE 0: the weights are asked for in front of the row's quantization; 1: behind it; 2: the first half of
   * the wavefront's rows in front, the other half behind. A template parameter: chosen at run time, the
   * places' loads end in different registers that are copied where the paths meet, which waits for every
   * load in front of the barrier; this way they stay in flight across it and each pass of the arithmetic
   * waits for its own. Which is fastest depends on the row length and the size (fused_weights_late): the
   * row's quantization wants its own loads back first and the weights' requests out early, and a wavefront
   * that issues sixteen loads in front of it is late for the barrier the workgroup waits at. */
  typename E::Wts W[NW];
  constexpr int HP = E::NP / 2; /* LATE == 2: the first half of a wavefront's passes in front, the rest behind */
  if constexpr (LATE == 0) {
#pragma unroll
    for (int i = 0; i < NW; ++i) E::load_w(W[i], wv[i], row0, 0, K);
  } else if constexpr (LATE == 2) {
#pragma unroll
    for (int i = 0; i < NW; ++i) E::template load_w<0, HP>(W[i], wv[i], row0, 0, K);
  }

  QView qa;
  qa.K = K;
  qa.q = (const int8_t *)ap;
  if (DT == HIPQ_Q4_0) {
    int8_t *q = (int8_t *)ap;
    uint32_t *meta = (uint32_t *)(ap + K);
    qa.meta = meta;
    qa.d = nullptr;
    qa.bsum = nullptr;
    qa.ql = qa.qh = nullptr;
    const int nb = K >> 5, sub = threadIdx.x & 7;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      if (32 * p >= nb) break; /* uniform */
      const int blk = (int)(threadIdx.x >> 3) + 32 * p;
      uint16_t dh;
      int qsum;
      const int packed = hipq_quantize_q8_0_lane(xs[p], dh, qsum);
      const int bsum = hipq_group_sum_i<8>(qsum);
      if (blk < nb) {
        *(int *)(q + blk * 32 + sub * 4) = packed;
        if (sub == 0) meta[blk] = (uint32_t)dh | ((uint32_t)(bsum & 0xffff) << 16);
      }
    }
  } else {
    int8_t *q = (int8_t *)ap;
    uint16_t *ql = (uint16_t *)(ap + K), *qh = (uint16_t *)(ap + K + (K >> 1));
    int16_t *bsum = (int16_t *)(ap + 2 * K);
    float *d = (float *)(ap + 2 * K + (K >> 3));
    qa.meta = nullptr;
    qa.d = d;
    qa.bsum = bsum;
    qa.ql = (const uint8_t *)ql;
    qa.qh = (const uint8_t *)qh;
    const int nsb = K >> 8;
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int sb = wave + WV * p;
      if (sb >= nsb) break; /* uniform per wavefront */
      hipq_quantize_q8_K_values < DT == HIPQ_Q4_K ? Q8K_DIGITS : Q8K_BYTES > (xs[p], 0, sb, sb, nsb, 0, q, d, bsum,
                                                                             nullptr, nullptr, ql, qh);
    }
  }
  if constexpr (LATE == 1) {
#pragma unroll
    for (int i = 0; i < NW; ++i) E::load_w(W[i], wv[i], row0, 0, K);
  } else if constexpr (LATE == 2) {
#pragma unroll
    for (int i = 0; i < NW; ++i) E::template load_w<HP, E::NP>(W[i], wv[i], row0, 0, K);
  }
  __syncthreads();

  typename E::Act A;
  E::load_act(A, qa, arow, 0, K);
  GemvOut o[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    typename E::Chain c = E::begin(arow, 0);
    E::compute(W[i], A, K, lds);
    hipq_wave_lds_sync();
    E::chain(c, K, lds);
    hipq_wave_lds_sync();
    o[i] = E::finish(c);
  }
  /* the results of the NW weights' row row0 + o[0].g sit in the same lane */
  if (o[0].valid && row0 + o[0].g < w.N) store(row0 + o[0].g, o);
}

template <int DT, int T, int G, int LATE, int FK>
__device__ __forceinline__ void gemv_fused_body(const WView &w, const float *__restrict__ x,
                                                float *__restrict__ C, int block) {
  const WView wv[1] = {w};
  gemv_fused_rows<DT, T, G, 1, LATE, FK>(wv, x, block, [&](int row, const GemvOut(&o)[1]) { C[row] = o[0].v; });
}

/* out[n] = silu(x . Wact[n]) * (x . Wmul[n]): the two projections of a gated MLP and the
 * SwiGLU between them and the down projection as one launch. A wavefront forms the same G
 * rows of both matrices (their loads in flight together) and the lane that ends up with
 * row n of the one also holds row n of the other. The activation is the framework's swiglu
 * (X = (Y / (1 + exp(-Y))) * Z in fp32, fallback_internal.cpp:417-423), applied by
 * SwiGLULayer::incremental_forwarding to the outputs of ffn_up (Y) and ffn_gate (Z)
 * (Applications/CausalLM/layers/swiglu.cpp:40-62, causal_lm.cpp:690-695). */
template <int DT, int T, int G, int LATE, int FK>
__global__ __launch_bounds__(256) void gemv_fused_swiglu_kernel(WView wact, WView wmul,
                                                                const float *__restrict__ x,
                                                                float *__restrict__ out) {
  const WView wv[2] = {wact, wmul};
  gemv_fused_rows<DT, T, G, 2, LATE, FK>(wv, x, (int)blockIdx.x, [&](int row, const GemvOut(&o)[2]) {
    const float y = o[0].v, z = o[1].v;
    out[row] = (y / (1.f + expf(-y))) * z;
  });
}

template <int DT, int T, int G, int LATE, int FK>
__global__ __launch_bounds__(256) void gemv_fused_kernel(WView w, const float *__restrict__ x,
                                                         float *__restrict__ C) {
  gemv_fused_body<DT, T, G, LATE, FK>(w, x, C, (int)blockIdx.x);
}
/* The same with WV wavefronts a workgroup: one workgroup a CU quantizes the row once where three of four
 * wavefronts each would quantize it three times (see launch_fused for where that pays). */
template <int DT, int T, int G, int WV, int LATE, int FK>
__global__ __launch_bounds__(64 * WV) void gemv_fused_wide_kernel(WView w, const float *__restrict__ x,
                                                                  float *__restrict__ C) {
  const WView wv[1] = {w};
  gemv_fused_rows<DT, T, G, 1, LATE, FK, WV>(wv, x, (int)blockIdx.x,
                                         [&](int row, const GemvOut(&o)[1]) { C[row] = o[0].v; });
}

/* Up to four weights of one format and K on the same row, one launch: the
 * workgroups of weight i are blocks end[i-1] .. end[i]-1 of the grid. */
constexpr int FUSED_MAXW = 4;
struct FusedMulti {
  WView w[FUSED_MAXW];
  float *C[FUSED_MAXW];
  int end[FUSED_MAXW];
};
template <int DT, int T, int G, int LATE, int FK>
__global__ __launch_bounds__(256) void gemv_fused_multi_kernel(FusedMulti mw, const float *__restrict__ x) {
  const int b = (int)blockIdx.x;
  int i = 0;
#pragma unroll
  for (int k = 0; k + 1 < FUSED_MAXW; ++k) i += b >= mw.end[k];
  const int first = i ? mw.end[i - 1] : 0;
  gemv_fused_body<DT, T, G, LATE, FK>(mw.w[i], x, mw.C[i], b - first);
}

/* The name a launch is noted under, with the instance's template arguments as numbers (what a kernel trace
 * prints): built once per instance. */
template <int FAMILY, int... V> const char *kernel_name(const char *base) { /* FAMILY: one number a kernel template */
  static const std::string name = [&] {
    std::string n = std::string(base) + "<";
    const int v[] = {V...};
    for (size_t i = 0; i < sizeof(v) / sizeof(v[0]); ++i) n += (i ? ", " : "") + std::to_string(v[i]);
    (void)FAMILY;
    return n + ">";
  }();
  return name.c_str();
}

/* Where a wavefront asks for its weights (gemv_fused_rows' LATE), by the row length and the weights of the
 * launch (all its matrices together). Measured with the usual row lengths as constants (us a call, in front /
 * behind / half and half): Q4_K 2048 x 4096 4.35 / 4.57 / 4.3, 4096 x 4096 5.35 / 5.25 / 5.2, 12288 x 4096
 * 8.1 / 8.1 / 7.65, 14336 x 4096 9.95 / 9.15 / 8.8, 24576 x 4096 13.3 / 13.7 / 12.65, 8192 x 3072 7.2 / 6.45 / 6.25,
 * 12288 x 2048 5.15 / 4.35 / 4.7, 16384 x 2048 6.65 / 5.65 / 6.3, 4096 x 2048 4.2 / 4.1 / 4.25; Q6_K 4096 x 4096
 * 5.75 / 5.85 / 5.0, 8192 x 4096 8.3 / 7.9 / 7.6; Q4_0 12288 x 4096 9.7 / 10.0 / 9.4, the C5 shapes (1024 .. 3072
 * rows of 1024 .. 3072) the same within 0.1 (in front 4.0-4.6); gate and up with the SwiGLU 11008 x 4096 13.9 /
 * 14.2 / 13.1, 8192 x 2048 7.45 / 6.4 / 6.9; Q, K, V of 4096 + 1024 + 1024 x 4096 6.7 / 6.5 / 6.3. */
static inline int fused_weights_late(int64_t K, int64_t weights) {
  if (K == 4096) return 2;
  if (weights < ((int64_t)1 << 24)) return 0;
  return K >= 3072 ? 2 : 1;
}

/* f(LATE, FK) with the two as compile-time constants. Rows of 16 lanes a row (under 2048 weights) have one
 * pass of weight rows a wavefront: no half and half. */
template <int T, typename F> void with_late(int late, int64_t K, F f) {
  auto go = [&](auto L) {
    if (T == 64 && K == 4096)
      f(L, std::integral_constant<int, T == 64 ? 4096 : 0>{});
    else if (T == 64 && K == 3072)
      f(L, std::integral_constant<int, T == 64 ? 3072 : 0>{});
    else if (T == 64 && K == 2048)
      f(L, std::integral_constant<int, T == 64 ? 2048 : 0>{});
    else if (T == 16 && K == 1024)
      f(L, std::integral_constant<int, T == 16 ? 1024 : 0>{});
    else
      f(L, std::integral_constant<int, 0>{});
  };
  if (late == 2 && T == 64)
    go(std::integral_constant<int, T == 64 ? 2 : 1>{});
  else if (late)
    go(std::integral_constant<int, 1>{});
  else
    go(std::integral_constant<int, 0>{});
}

template <int DT, int T, int G>
int launch_fused_many(int count, const hipq_weight *const *w, const float *x, float *const *C, hipStream_t s) {
  FusedMulti mw;
  int blocks = 0;
  int64_t weights = 0;
  for (int i = 0; i < FUSED_MAXW; ++i) {
    const int j = i < count ? i : count - 1;
    mw.w[i] = wview(w[j]);
    mw.C[i] = C[j];
    if (i < count) blocks += (int)((w[i]->N + 4 * G - 1) / (4 * G)), weights += w[i]->N * w[i]->K;
    mw.end[i] = blocks;
  }
  const size_t lds = fused_act_bytes<DT>((int)w[0]->K) + 4 * GemvLds<DT, 1, G, false>::DWORDS * sizeof(uint32_t);
  with_late<T>(fused_weights_late(w[0]->K, weights), w[0]->K, [&](auto L, auto FK) {
    hipq::launch_kernel(kernel_name<1, DT, T, G, decltype(L)::value, decltype(FK)::value>("gemv_fused_multi_kernel"),
                        (gemv_fused_multi_kernel<DT, T, G, decltype(L)::value, decltype(FK)::value>),
                        dim3((unsigned)blocks), dim3(256), lds, s, mw, x);
  });
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int T, int G, int WV>
int launch_fused_wide(const hipq_weight *w, const float *x, float *C, hipStream_t s) {
  const unsigned grid = (unsigned)((w->N + WV * G - 1) / (WV * G));
  const size_t lds = fused_act_bytes<DT>((int)w->K) + WV * GemvLds<DT, 1, G, false>::DWORDS * sizeof(uint32_t);
  with_late<T>(fused_weights_late(w->K, w->N * w->K), w->K, [&](auto L, auto FK) {
    hipq::launch_kernel(kernel_name<2, DT, T, G, WV, decltype(L)::value, decltype(FK)::value>("gemv_fused_wide_kernel"),
                        (gemv_fused_wide_kernel<DT, T, G, WV, decltype(L)::value, decltype(FK)::value>),
                        dim3(grid), dim3(64 * WV), lds, s, wview(w), x, C);
  });
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int T, int G>
int launch_fused_one(const hipq_weight *w, const float *x, float *C, hipStream_t s) {
  const unsigned grid = (unsigned)((w->N + 4 * G - 1) / (4 * G));
  const size_t lds = fused_act_bytes<DT>((int)w->K) + 4 * GemvLds<DT, 1, G, false>::DWORDS * sizeof(uint32_t);
  with_late<T>(fused_weights_late(w->K, w->N * w->K), w->K, [&](auto L, auto FK) {
    constexpr int LATE = decltype(L)::value == 2 && G < 2 ? 0 : decltype(L)::value; /* half and half takes two passes */
    hipq::launch_kernel(kernel_name<3, DT, T, G, LATE, decltype(FK)::value>("gemv_fused_kernel"),
                        (gemv_fused_kernel<DT, T, G, LATE, decltype(FK)::value>), dim3(grid),
                        dim3(256), lds, s, wview(w), x, C);
  });
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int T, int G, int GPW>
int launch_stream(const hipq_weight *w, const QAct *qa, float *C, hipStream_t s) {
  const int rows_per_block = 4 * G * GPW;
  const unsigned grid = (unsigned)((w->N + rows_per_block - 1) / rows_per_block);
  const size_t lds = 4 * GemvLds<DT, 1, G, false>::DWORDS * sizeof(uint32_t);
  constexpr int USUAL = T == 64 ? 4096 : 1024; /* the row length that has an instance of its own */
  if (w->K == USUAL)
    hipq::launch_kernel(kernel_name<4, DT, T, G, GPW, USUAL>("gemv_stream_kernel"), (gemv_stream_kernel<DT, T, G, GPW, USUAL>), dim3(grid), dim3(256),
                        lds, s, wview(w), qview(*qa), C);
  else
    hipq::launch_kernel(kernel_name<4, DT, T, G, GPW, 0>("gemv_stream_kernel"), (gemv_stream_kernel<DT, T, G, GPW, 0>), dim3(grid), dim3(256), lds,
                        s, wview(w), qview(*qa), C);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int DT, int T, int R, int G, bool PW>
int launch_one(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
               hipStream_t s) {
  const unsigned grid = (unsigned)((w->N + 4 * G - 1) / (4 * G));
  const size_t lds = 4 * GemvLds<DT, R, G, PW>::DWORDS * sizeof(uint32_t);
  constexpr int USUAL = T == 64 ? 4096 : 1024; /* the row length that has an instance of its own */
  if (w->K == USUAL)
    hipq::launch_kernel(kernel_name<5, DT, T, R, G, PW, USUAL>("gemv_kernel"), (gemv_kernel<DT, T, R, G, PW, USUAL>), dim3(grid), dim3(256), lds, s,
                        wview(w), qview(*qa), M, pair_rows, C, ldc);
  else if (R == 1 && T == 64 && w->K == 2048) /* one row: two more lengths */
    hipq::launch_kernel(kernel_name<5, DT, T, R, G, PW, 2048>("gemv_kernel"), (gemv_kernel<DT, T, R, G, PW, R == 1 && T == 64 ? 2048 : 0>), dim3(grid),
                        dim3(256), lds, s, wview(w), qview(*qa), M, pair_rows, C, ldc);
  else if (R == 1 && T == 64 && w->K == 3072)
    hipq::launch_kernel(kernel_name<5, DT, T, R, G, PW, 3072>("gemv_kernel"), (gemv_kernel<DT, T, R, G, PW, R == 1 && T == 64 ? 3072 : 0>), dim3(grid),
                        dim3(256), lds, s, wview(w), qview(*qa), M, pair_rows, C, ldc);
  else
    hipq::launch_kernel(kernel_name<5, DT, T, R, G, PW, 0>("gemv_kernel"), (gemv_kernel<DT, T, R, G, PW, 0>), dim3(grid), dim3(256), lds, s,
                        wview(w), qview(*qa), M, pair_rows, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* Largest group size not above gmax that still gives ~6000 wavefronts. */
int pick_group(int64_t N, int gmax) {
  /* measured: 4 rows per wavefront is best from N = 8192 up to the 151936-row
   * lm_head; smaller matrices want more, shorter wavefronts */
  int g = N >= 8192 ? 4 : (N >= 2048 ? 2 : 1);
  return g < gmax ? g : gmax;
}

template <int DT, int T, int G>
int launch_fused_swiglu_one(const hipq_weight *wa, const hipq_weight *wm, const float *x, float *out,
                            hipStream_t s) {
  const unsigned grid = (unsigned)((wa->N + 4 * G - 1) / (4 * G));
  const size_t lds = fused_act_bytes<DT>((int)wa->K) + 4 * GemvLds<DT, 1, G, false>::DWORDS * sizeof(uint32_t);
  with_late<T>(fused_weights_late(wa->K, 2 * wa->N * wa->K), wa->K, [&](auto L, auto FK) {
    hipq::launch_kernel(kernel_name<6, DT, T, G, decltype(L)::value, decltype(FK)::value>("gemv_fused_swiglu_kernel"),
                        (gemv_fused_swiglu_kernel<DT, T, G, decltype(L)::value, decltype(FK)::value>),
                        dim3(grid), dim3(256), lds, s, wview(wa), wview(wm), x, out);
  });
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* the shapes of launch_fused for twice the rows (two matrices a wavefront) */
template <int DT>
int launch_fused_swiglu(const hipq_weight *wa, const hipq_weight *wm, const float *x, float *out, hipStream_t s) {
  const int64_t units = wa->K / GemvRec<DT, false>::UNIT;
  /* a wavefront forms G rows of each matrix: half the group of a single matrix with as many rows */
  const int g = pick_group(2 * wa->N, 8) / 2;
  if (units < 64) return launch_fused_swiglu_one<DT, 16, 4>(wa, wm, x, out, s);
  if (g >= 4) return launch_fused_swiglu_one<DT, 64, 4>(wa, wm, x, out, s);
  if (g == 2) return launch_fused_swiglu_one<DT, 64, 2>(wa, wm, x, out, s);
  return launch_fused_swiglu_one<DT, 64, 1>(wa, wm, x, out, s);
}

/* One activation row: the decode shape, tuned for parallelism. */
template <int DT>
int launch_m1(const hipq_weight *w, const QAct *qa, float *C, int64_t ldc, hipStream_t s) {
  const int64_t units = w->K / GemvRec<DT, false>::UNIT;
  /* measured on lm_head-sized matrices (N = 151936): two groups per wavefront with
   * the next group's loads in flight gain 3 % (Q4_K) to 20 % (Q4_0) over the plain kernel whose loads the
   * waits cannot count (any row length); Q6_K and smaller matrices are better off with more, shorter
   * wavefronts, and so are rows of 4096 now that the plain kernel's waits count every load (us a call with
   * the quantizer's launch, streamed -> plain: Q4_K 32768 x 4096 17.6 -> 16.1, 65536 29.0 -> 26.4, 151936
   * 57.2 -> 53.9; Q4_0 32768 20.1 -> 17.7, 151936 59.0 -> 57.0), and rows of 2048 and 3072, which the plain kernel
   * has as constants for one row too (Q4_K 151936 x 2048 35 -> 29, 65536 x 2048 18.6 -> 15.5, 151936 x 3072 47.7 -> 46.2;
   * Q4_0 151936 x 2048 39.7 -> 31) */
  if (DT != HIPQ_Q6_K && w->N >= 32768 && w->K < HIPQ_KCHUNK && w->K != 2048 && w->K != 3072 && units >= 64)
    return launch_stream<DT, 64, 4, 2>(w, qa, C, s);
  /* the same for short rows (16 lanes a row, four rows side by side, eight a group): a wavefront of
   * the plain kernel below would have four short rows for all its work. Kernel us, plain -> streamed:
   * Q4_K 151936 x 1024 38.0 -> 31.9, 151936 x 256 27.9 -> 21.8, 65536 x 512 13.2 -> 10.7, 32768 x 1024
   * 9.4 -> 8.0; Q4_0 32768 x 1024 8.4 -> 6.9 (wider Q4_0 matrices take the few-rows kernel); Q6_K is
   * the slower for it (151936 x 1024 34.6 -> 38.0) and stays */
  if (DT != HIPQ_Q6_K && w->N >= 32768 && w->K <= HIPQ_KCHUNK && units < 64)
    return DT == HIPQ_Q4_0 ? launch_stream<DT, 16, 8, 2>(w, qa, C, s) : launch_stream<DT, 16, 8, 4>(w, qa, C, s);
  if (units < 64) { /* short rows: 16 lanes per row, 4 rows streamed at once */
    if (pick_group(w->N, 8) == 8) return launch_one<DT, 16, 1, 8, false>(w, qa, 1, 0, C, ldc, s);
    return launch_one<DT, 16, 1, 4, false>(w, qa, 1, 0, C, ldc, s);
  }
  switch (pick_group(w->N, 8)) {
  case 8:
    return launch_one<DT, 64, 1, 8, false>(w, qa, 1, 0, C, ldc, s);
  case 4:
    return launch_one<DT, 64, 1, 4, false>(w, qa, 1, 0, C, ldc, s);
  case 2:
    return launch_one<DT, 64, 1, 2, false>(w, qa, 1, 0, C, ldc, s);
  default:
    /* Q4_0's fp32 chain has one step per 32 weights: keep two rows per pass */
    if (DT == HIPQ_Q4_0) return launch_one<DT, 64, 1, 2, false>(w, qa, 1, 0, C, ldc, s);
    return launch_one<DT, 64, 1, 1, false>(w, qa, 1, 0, C, ldc, s);
  }
}

/* The shapes of launch_m1 below its streaming case, on the fp32 row. */
template <int DT> int launch_fused(const hipq_weight *w, const float *x, float *C, hipStream_t s) {
  const int64_t units = w->K / GemvRec<DT, false>::UNIT;
  if (units < 64) {
    if (pick_group(w->N, 8) == 8) return launch_fused_one<DT, 16, 8>(w, x, C, s);
    return launch_fused_one<DT, 16, 4>(w, x, C, s);
  }
  if constexpr (DT == HIPQ_Q4_K) {
    /* Workgroups of twelve wavefronts quantize the row once where three of four wavefronts each would
     * quantize it three times. With rows of 4096 and every load counted by the waits, two rows a wavefront
     * (24 a workgroup) are the fastest form wherever the workgroups fill the CUs' rounds evenly (us a call,
     * four wavefronts of four rows / twelve of four / twelve of two: 3072 rows 4.6 / 6.1 / 4.5, 5120 5.85 / 6.4 /
     * 4.75, 6144 5.8 / 6.4 / 4.9, 11008 7.6 / 7.5 / 7.05, 12288 7.35 / 7.65 / 7.1, 18432 10.65 / 11.8 / 9.35, 24576
     * 12.6 / 12.7 / 11.5), and four wavefronts of four rows where the last round would be short (7168 5.95 / 6.55 /
     * 6.75, 8192 5.9 / 6.65 / 6.9, 20480 10.9 / 11.85 / 11.35). Other row lengths keep the form measured for them
     * (twelve wavefronts of four rows up to one round: 12288 x 2048 6.1 -> 5.6 when it was introduced). */
    if (w->K == HIPQ_KCHUNK && w->N >= 2048) {
      const int64_t wgs = (w->N + 23) / 24, rest = wgs % 256;
      if (wgs <= 256 || rest == 0 || rest >= 128) return launch_fused_wide<DT, 64, 2, 12>(w, x, C, s);
      return launch_fused_one<DT, 64, 4>(w, x, C, s);
    }
    /* shorter rows: twelve wavefronts of two rows up to one round of them (6144 x 2048 4.85 -> 4.1 us a call,
     * 4096 x 2048 4.3 -> 4.1, 3072 x 3072 5.3 -> 5.05), of four rows up to one round of those */
    if (w->N >= 2048 && (w->N + 23) / 24 <= 256) return launch_fused_wide<DT, 64, 2, 12>(w, x, C, s);
    if (pick_group(w->N, 8) == 4 && (w->N + 47) / 48 <= 256) return launch_fused_wide<DT, 64, 4, 12>(w, x, C, s);
  }
  /* Q4_0: four rows a wavefront from 4096 rows on (4096 x 4096 6.65 -> 6.25 us a call, 6144 x 4096 7.65 -> 7.3,
   * 4096 x 2048 4.4 -> 4.15, 6144 x 2048 4.9 -> 4.6) */
  if (DT == HIPQ_Q4_0 && w->N >= 4096) return launch_fused_one<DT, 64, 4>(w, x, C, s);
  switch (pick_group(w->N, 8)) {
  case 8:
    return launch_fused_one<DT, 64, 8>(w, x, C, s);
  case 4:
    return launch_fused_one<DT, 64, 4>(w, x, C, s);
  case 2:
    return launch_fused_one<DT, 64, 2>(w, x, C, s);
  default:
    /* Q4_0 rows are short work for a wavefront: two of them, unless that leaves CUs without a workgroup (1024 rows
     * of 3072: 4.6 -> 4.4 us a call, of 4096: 5.5 -> 5.1; 1536 rows of 3072: 4.6 against 4.8) */
    if (DT == HIPQ_Q4_0 && w->N > 1024) return launch_fused_one<DT, 64, 2>(w, x, C, s);
    return launch_fused_one<DT, 64, 1>(w, x, C, s);
  }
}

template <int DT>
int launch_fused_multi(int count, const hipq_weight *const *w, const float *x, float *const *C, hipStream_t s) {
  int64_t n = 0;
  for (int i = 0; i < count; ++i) n += w[i]->N;
  const int64_t units = w[0]->K / GemvRec<DT, false>::UNIT;
  const int g = pick_group(n, 8);
  if (units < 64) {
    if (g == 8) return launch_fused_many<DT, 16, 8>(count, w, x, C, s);
    return launch_fused_many<DT, 16, 4>(count, w, x, C, s);
  }
  if (g == 8) return launch_fused_many<DT, 64, 8>(count, w, x, C, s);
  if (g == 4) return launch_fused_many<DT, 64, 4>(count, w, x, C, s);
  if (g == 2 || DT == HIPQ_Q4_0) return launch_fused_many<DT, 64, 2>(count, w, x, C, s);
  return launch_fused_many<DT, 64, 1>(count, w, x, C, s);
}

/* 2..8 activation rows in one pass (small prefill chunks, leftover rows). */
template <int DT>
int launch_mr(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
              hipStream_t s) {
  constexpr bool K4 = DT == HIPQ_Q4_K;
  if (M == 2) return launch_one<DT, 64, 2, (K4 ? 4 : 2), false>(w, qa, M, 0, C, ldc, s);
  if (M == 3) return launch_one<DT, 64, 4, 2, false>(w, qa, M, 0, C, ldc, s);
  if (M == 4) return launch_one<DT, 64, 4, 2, K4>(w, qa, M, pair_rows, C, ldc, s);
  return launch_one<DT, 64, 8, 1, K4>(w, qa, M, pair_rows, C, ldc, s);
}

} // namespace

namespace hipq {

int launch_gemv(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
                hipStream_t s) {
  if (M < 1 || M > 8) return fail(HIPQ_ERR_INVALID_ARGUMENT, "gemv handles 1..8 rows, got %d", M);
  switch (w->dtype) {
  case HIPQ_Q4_0:
    return M == 1 ? launch_m1<HIPQ_Q4_0>(w, qa, C, ldc, s)
                  : launch_mr<HIPQ_Q4_0>(w, qa, M, pair_rows, C, ldc, s);
  case HIPQ_Q4_K:
    return M == 1 ? launch_m1<HIPQ_Q4_K>(w, qa, C, ldc, s)
                  : launch_mr<HIPQ_Q4_K>(w, qa, M, pair_rows, C, ldc, s);
  case HIPQ_Q6_K:
    return M == 1 ? launch_m1<HIPQ_Q6_K>(w, qa, C, ldc, s)
                  : launch_mr<HIPQ_Q6_K>(w, qa, M, pair_rows, C, ldc, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", w->dtype);
}

/* Rows of one chunk, 16-byte aligned, and matrices below 32768 rows (the sizes that
 * launch_m1 does not stream): beyond that the quantizer's launch is a few per cent of
 * the GEMV and thousands of workgroups quantizing the row again cost more (measured
 * on a 151936 x 4096 Q6_K matrix: 92.9 us against 81.6 us with two launches). */
bool gemv_fuses_quantizer(const hipq_weight *w, const float *x) {
  return w->K <= HIPQ_KCHUNK && w->N < 32768 && ((uintptr_t)x & 15) == 0;
}

bool gemv_fuses_quantizer_multi(int count, const hipq_weight *const *w, const float *x) {
  if (count < 1 || count > FUSED_MAXW) return false;
  int64_t n = 0;
  for (int i = 0; i < count; ++i) {
    if (w[i]->dtype != w[0]->dtype || w[i]->K != w[0]->K || !gemv_fuses_quantizer(w[i], x)) return false;
    n += w[i]->N;
  }
  return n < 32768;
}

int launch_gemv_fused_multi(int count, const hipq_weight *const *w, const float *x, float *const *C,
                            hipStream_t s) {
  if (!gemv_fuses_quantizer_multi(count, w, x))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "these matrices do not take the GEMV that quantizes its own row");
  switch (w[0]->dtype) {
  case HIPQ_Q4_0:
    return launch_fused_multi<HIPQ_Q4_0>(count, w, x, C, s);
  case HIPQ_Q4_K:
    return launch_fused_multi<HIPQ_Q4_K>(count, w, x, C, s);
  case HIPQ_Q6_K:
    return launch_fused_multi<HIPQ_Q6_K>(count, w, x, C, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", w[0]->dtype);
}

bool gemv_fuses_swiglu(const hipq_weight *wa, const hipq_weight *wm, const float *x) {
  return wa->dtype == wm->dtype && wa->K == wm->K && wa->N == wm->N && gemv_fuses_quantizer(wa, x) &&
         2 * wa->N < 32768;
}

int launch_gemv_fused_swiglu(const hipq_weight *wa, const hipq_weight *wm, const float *x, float *out,
                             hipStream_t s) {
  if (!gemv_fuses_swiglu(wa, wm, x))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "these matrices do not take the fused gated-MLP GEMV");
  switch (wa->dtype) {
  case HIPQ_Q4_0:
    return launch_fused_swiglu<HIPQ_Q4_0>(wa, wm, x, out, s);
  case HIPQ_Q4_K:
    return launch_fused_swiglu<HIPQ_Q4_K>(wa, wm, x, out, s);
  case HIPQ_Q6_K:
    return launch_fused_swiglu<HIPQ_Q6_K>(wa, wm, x, out, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", wa->dtype);
}

/* out[m][n] = (y / (1 + exp(-y))) * z, elementwise (the same activation for M > 1 rows) */
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const float *__restrict__ y, const float *__restrict__ z,
                                                          int64_t n_total, int64_t N, int64_t ldo,
                                                          float *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_total) return;
  const float yv = y[i], zv = z[i];
  out[(i / N) * ldo + i % N] = (yv / (1.f + expf(-yv))) * zv;
}

int launch_swiglu_rows(const float *y, const float *z, int64_t M, int64_t N, float *out, int64_t ldo, hipStream_t s) {
  const int64_t n = M * N;
  hipq::launch_kernel("swiglu_rows_kernel", swiglu_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, y, z, n, N, ldo, out);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_gemv_fused(const hipq_weight *w, const float *x, float *C, hipStream_t s) {
  if (!gemv_fuses_quantizer(w, x))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "this matrix does not take the GEMV that quantizes its own row");
  switch (w->dtype) {
  case HIPQ_Q4_0:
    return launch_fused<HIPQ_Q4_0>(w, x, C, s);
  case HIPQ_Q4_K:
    return launch_fused<HIPQ_Q4_K>(w, x, C, s);
  case HIPQ_Q6_K:
    return launch_fused<HIPQ_Q6_K>(w, x, C, s);
  }
  return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", w->dtype);
}

} // namespace hipq
