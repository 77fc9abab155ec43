// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hipq_internal.h
 * @brief  Shared declarations of the gfx950 quantized-matmul library: device
 *         data layouts, launch entry points of each kernel family and the
 *         device-side helpers (wave reductions over DPP, int8 dot, half
 *         conversion) they have in common.
 */
#ifndef HIPQ_INTERNAL_H
#define HIPQ_INTERNAL_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <vector>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "hipq.h"

/* ------------------------------------------------------------------------- */
/* Device-resident weight matrix (W^T, N rows of K quantized values).         */
/*                                                                            */
/* The ggml array-of-structs blocks are split once, at creation, into planes  */
/* so that every lane of a wavefront can issue aligned 128-bit loads:         */
/*   Q4_0: qs [N][K/2]  (16 B per 32-block, nibble order of block_q4_0)       */
/*         d  [N][K/32] fp16                                                  */
/*   Q4_K: qs [N][K/2]  (128 B per super-block: sub-block j = bytes 16j..16j+15, */
/*                      weight 2i low / 2i+1 high nibble of byte i)             */
/*         hdr[N][K/256][16] = {fp16 d, fp16 dmin, sm[8], ml[4]}: the 6-bit     */
/*                      scales sc_j and mins m_j of block_q4_K regrouped so that */
/*                      byte sm[j] = sc_j | (m_j >> 4) << 6 and byte ml[k] =     */
/*                      (m_k & 15) | (m_(k+4) & 15) << 4. A GEMV lane takes the  */
/*                      scale and min of ONE sub-block with three shifts; the    */
/*                      matrix kernels take all eight as bytes of two words      */
/*   Q6_K: qs [2][N][K/4] (ql in two planes, 64 B per super-block each: unit  */
/*                      uu = half*2 + hl holds bytes half*64 + hl*16 .. +15 of  */
/*                      block_q6_K::ql in the first and those 32 further on in   */
/*                      the second)                                              */
/*         qh [N][K/4]  (64 B per super-block, same byte order)               */
/*         sc [N][K/16] int8, regrouped per super-block as [unit u][group g]  */
/*                      = scales[(u>>1)*8 + g*2 + (u&1)]                      */
/*         d  [N][K/256] fp16                                                 */
/* The total size equals the packed ggml size; nothing is expanded in HBM.    */
/*                                                                             */
/* Q4_K expert weights of a mixture-of-experts block that runs on the matrix   */
/* cores are re-laid out once more, by tiles of 32 rows (rows padded to 32),   */
/* 4608 bytes per tile and super-block, [N/32][K/256]{qs, hdr}:                */
/*   qs  [4][64][16 B]: for load i of lane (n, g) the two 8-byte halves g of    */
/*       sub-blocks 2i and 2i+1 of row n -- the 16 bytes the lane feeds into    */
/*       two matrix steps, consecutive lanes consecutive in memory              */
/*   hdr [32][16 B]: the headers of the tile's rows, right behind their nibbles */
/*       (a wavefront's stream over a tile is one run of consecutive memory;    */
/*       hipq_weight.hdr points at the first header, 4096 bytes behind qs)      */
/* Such a weight serves the expert kernels only.                               */
/* ------------------------------------------------------------------------- */
struct hipq_weight {
  int dtype;
  int device;
  int expert_tiles; /* Q4_K only: re-laid out for the matrix-core expert kernels (see below) */
  int64_t N, K;
  uint8_t *base;   /* one allocation holding all planes */
  size_t bytes;
  const uint8_t *qs;
  const uint8_t *qh;
  const uint8_t *hdr;
  const int8_t *sc;
  const uint16_t *d;
  /* Built by the first prefill product of the weight (ensure_gemm_tiles): a second copy by
   * tiles of 32 rows, in the order the wavefronts of the prefill GEMM load it, so that each
   * of their 128-bit load instructions covers 1 KB of consecutive memory.
   * Q4_K:
   *   gt_qs  [N/32][K/256][4][64][16 B]: load i of lane (n, g) = sub-block 4g + i of row n
   *   gt_hdr [N/32][K/256][32][16 B]
   * Q6_K: lane (n, g) owns half g (128 weights) of row n's super-block, eight steps of 16
   *   weights with one scale each:
   *   gt_qs  [N/32][K/256][4][64][16 B]: load i = steps 2i, 2i+1; per step 8 bytes, weight
   *          2k / 2k+1 of the step's 16 in the low / high nibble of byte k (low four bits)
   *   gt_qh  [N/32][K/256][2][64][16 B]: load i = steps 4i .. 4i+3; per step 4 bytes, byte k =
   *          bits 4-5 of weights 2k, 2k+8, 2k+1, 2k+9 (two bits each, in that order)
   *   gt_hdr [N/32][K/256][64][16 B]: the lane's eight int8 scales, then the fp16 d */
  uint8_t *gt_base;
  const uint8_t *gt_qs, *gt_qh, *gt_hdr;
};

/* Plain-data view of a weight passed to kernels by value. */
struct WView {
  const uint8_t *qs;
  const uint8_t *qh;
  const uint8_t *hdr;
  const int8_t *sc;
  const uint16_t *d;
  int N, K;
};
static inline WView wview(const hipq_weight *w) {
  WView v;
  v.qs = w->qs;
  v.qh = w->qh;
  v.hdr = w->hdr;
  v.sc = w->sc;
  v.d = w->d;
  v.N = (int)w->N;
  v.K = (int)w->K;
  return v;
}

/* ------------------------------------------------------------------------- */
/* Internal (device) form of quantized activations, structure of arrays.      */
/*   Q8_0: q [M][K] int8; meta [M][K/32] = fp16 d bits | (int16 sum of the    */
/*         block's 32 quants) << 16                                           */
/*   Q8_K: q [M][K] int8; d [M][K/256] fp32; bsum [M][K/16] int16;            */
/*         ql, qh [M][K/2]: the same values split into 4-bit digits,           */
/*         q = 16 * (qh - 8) + ql, element 2i in the low nibble of byte i      */
/* The quantizers can alternatively emit the canonical ggml blocks.           */
/* ------------------------------------------------------------------------- */
struct QAct {
  int8_t *q;
  uint32_t *meta; /* Q8_0 */
  float *d;       /* Q8_K */
  int16_t *bsum;  /* Q8_K */
  uint8_t *ql;    /* Q8_K */
  uint8_t *qh;    /* Q8_K */
  int M, K;
};
size_t qact_bytes(int dtype_is_k, int64_t M, int64_t K);
QAct qact_carve(int dtype_is_k, void *mem, int64_t M, int64_t K);

/* ------------------------------------------------------------------------- */
/* Q8_K activations in the form the Q4_K prefill GEMM copies straight from    */
/* HBM into LDS, tiled by 128 rows (mt = m / 128, rows padded to 128):         */
/*   qt   [mt][K/128][16384]: one 128-row x 128-deep stage, laid out as        */
/*        [m%128/32][step 4][g 2][m%32][16 bytes]: the 16-byte operands in the  */
/*        order the lanes of the 32x32x32 int8 matrix instruction take them.    */
/*        Lane group g covers sub-blocks 4g .. 4g+3 of the super-block, two     */
/*        steps each (first, second 16 values); an operand holds its 16 values   */
/*        as the 8 even then the 8 odd ones (as the weights' nibbles unpack)     */
/*   amin [mt][K/256][128][16] fp16: per row and super-block the eight         */
/*        sub-block sums (bsum[2j] + bsum[2j+1]) split into a part in 0..63    */
/*        (first 8) and a multiple of 64 (last 8), both exact in fp16          */
/*   dAt  [mt][K/256][128] fp32: the block scales d                            */
/* ------------------------------------------------------------------------- */
struct QActTiled {
  int8_t *qt;
  uint16_t *amin;
  float *dAt;
  int M, K, mtiles;
};
size_t qact_tiled_bytes(int64_t M, int64_t K);
QActTiled qact_tiled_carve(void *mem, int64_t M, int64_t K);

namespace hipq {

/* error plumbing (api.hip) */
int fail(int code, const char *fmt, ...);

/* Kernel timing (hipq_launch_timing_begin / _end of include/hipq.h): while the calling thread
 * has it switched on, every launch made through launch_kernel attaches a start and a stop event of
 * its own to the dispatch, which then hold the kernel's own start and end (no marker packets in
 * the stream between the kernels), and notes which kernel it was. Off otherwise: one thread-local
 * load per launch. */
struct LaunchLog {
  bool on = false;
  int count = 0, dropped = 0;
  std::vector<hipEvent_t> ev;     /* 2 per launch: start, stop */
  std::vector<const char *> fn;   /* the kernel as its launch site names it (a string literal) */
};
extern thread_local LaunchLog launch_log;
template <typename... KArgs, typename... Args>
inline void launch_kernel(const char *name, void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s,
                          Args... args) {
  LaunchLog &lg = launch_log;
  if (lg.on && (size_t)(2 * lg.count + 1) < lg.ev.size()) {
    hipExtLaunchKernelGGL(kernel, grid, block, lds, s, lg.ev[2 * lg.count], lg.ev[2 * lg.count + 1], 0, args...);
    lg.fn[lg.count++] = name;
    return;
  }
  if (lg.on) ++lg.dropped;
  hipLaunchKernelGGL(kernel, grid, block, lds, s, args...);
}
#define HIPQ_HIP(call)                                                        \
  do {                                                                        \
    hipError_t e_ = (call);                                                   \
    if (e_ != hipSuccess)                                                     \
      return ::hipq::fail(HIPQ_ERR_RUNTIME, "%s failed: %s (%s:%d)", #call,   \
                          hipGetErrorString(e_), __FILE__, __LINE__);         \
  } while (0)

/* quantize.hip ------------------------------------------------------------ */
/* Rows [0, M) of A (row stride lda). `canonical_out` != nullptr writes ggml
 * blocks there, otherwise the internal planes of `qa` are written.
 * mat_rows: rows [0, mat_rows) use the 4-row ("MAT") Q8_K semantics, the rest
 * the row semantics. */
int launch_quantize_q8_0(const float *A, int64_t M, int64_t K, int64_t lda,
                         const QAct *qa, void *canonical_out, hipStream_t s);
int launch_quantize_q8_K(const float *A, int64_t M, int64_t K, int64_t lda,
                         int64_t mat_rows, const QAct *qa, void *canonical_out,
                         hipStream_t s);
/* Row quantizer into a QAct whose planes take the form the grouped MFMA expert
 * kernels read: q row-major with every 16-value group stored as its 8 even then
 * its 8 odd values, d as usual, and in place of bsum 16 fp16 per super-block:
 * the eight sub-block sums split into a part in 0..63 (first 8) and a multiple
 * of 64 (last 8). ql / qh are not written. */
int launch_quantize_q8_K_rowmma(const float *A, int64_t M, int64_t K, int64_t lda, const QAct *qa,
                                hipStream_t s, int64_t mat_rows = 0);
/* the values of launch_quantize_q8_K, written in the tiled form; rows M .. 128 * mtiles
 * are zero-filled */
int launch_quantize_q8_K_tiled(const float *A, int64_t M, int64_t K, int64_t lda,
                               int64_t mat_rows, const QActTiled *qa, hipStream_t s);

/* gemv.hip ---------------------------------------------------------------- */
/* C[m][n] for m < M <= 8: one pass over the weights, M activation rows.
 * Rows below pair_rows use the reference GEMM kernel's fp32 order (Q4_K). */
/* one fp32 activation row, quantized inside the GEMV's workgroups (small matrices) */
bool gemv_fuses_quantizer(const hipq_weight *w, const float *x);
int launch_gemv_fused(const hipq_weight *w, const float *x, float *C, hipStream_t s);
/* the same for up to four weights of one format and K, one launch */
bool gemv_fuses_quantizer_multi(int count, const hipq_weight *const *w, const float *x);
int launch_gemv_fused_multi(int count, const hipq_weight *const *w, const float *x, float *const *C,
                            hipStream_t s);
/* out = swiglu(x . Wact, x . Wmul), one row, one launch; and the activation alone for M rows */
bool gemv_fuses_swiglu(const hipq_weight *wa, const hipq_weight *wm, const float *x);
int launch_gemv_fused_swiglu(const hipq_weight *wa, const hipq_weight *wm, const float *x, float *out,
                             hipStream_t s);
int launch_swiglu_rows(const float *y, const float *z, int64_t M, int64_t N, float *out, int64_t ldo, hipStream_t s);
int launch_gemv(const hipq_weight *w, const QAct *qa, int M, int pair_rows,
                float *C, int64_t ldc, hipStream_t s);

/* gemm.hip ---------------------------------------------------------------- */
int launch_gemm(const hipq_weight *w, const QAct *qa, int M, float *C,
                int64_t ldc, hipStream_t s);
/* up to four Q4_0 weights of one K against the same quantized rows, one launch */
int launch_gemm_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, float *const *C,
                      const int64_t *ldc, hipStream_t s);
/* gemm_q4k.hip: Q4_K with the sub-block scales folded into two int8 digit planes */
int launch_gemm_q4k_multi(int count, const hipq_weight *const *w, const QActTiled *qa, int M, float *const *C,
                          const int64_t *ldc, hipStream_t s);
int launch_gemm_q6k(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc, hipStream_t s,
                    void *partials = nullptr);
size_t gemm_q6k_split_bytes(const hipq_weight *w, int64_t M);
/* partials: gemm_q4k_split_bytes(w, M) bytes of device memory (or null): with few tiles the product
 * is formed in parts of K that run side by side and are then added */
int launch_gemm_q4k(const hipq_weight *w, const QActTiled *qa, int M, float *C,
                    int64_t ldc, hipStream_t s, void *partials = nullptr);
size_t gemm_q4k_split_bytes(const hipq_weight *w, int64_t M);
/* gemm_rows_q4k.hip: Q4_K for a few rows on the matrix cores with the reference's bits; fits: the row
 * counts and shapes that should take it (up to 16 rows, in passes of up to 8 for the launcher); qa in
 * the form of launch_quantize_q8_K_rowmma, the first pair_rows rows under the 4-row quantizer's rule;
 * the weight with its tile copy (ensure_gemm_tiles) */
bool gemm_rows_q4k_fits(const hipq_weight *w, int64_t M);
int launch_gemm_rows_q4k(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
                         hipStream_t s);
/* up to four weights of one K against the same rows in one launch (the column tiles side by side in the grid) */
bool gemm_rows_q4k_fits_multi(int count, const hipq_weight *const *w, int64_t M);
int launch_gemm_rows_q4k_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, int pair_rows,
                               float *const *C, const int64_t *ldc, hipStream_t s);

/* gemm_rows_q40.hip: Q4_0 for a few rows on the matrix cores with the reference's bits (rows are
 * independent in this format); fits: the row counts and shapes that should take it; qa in the form
 * of launch_quantize_q8_0; the weight's planes as they are */
bool gemm_rows_q40_fits(const hipq_weight *w, int64_t M);
int launch_gemm_rows_q40(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc, hipStream_t s);
/* up to four weights of one K against the same rows in one launch (the column tiles side by side in the grid) */
bool gemm_rows_q40_fits_multi(int count, const hipq_weight *const *w, int64_t M);
int launch_gemm_rows_q40_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, float *const *C,
                               const int64_t *ldc, hipStream_t s);
/* the same on the fp32 rows themselves (the workgroups quantize them: no quantizer launch, no workspace),
 * for small launches; fuses: whether a product should take it */
bool gemm_rows_q40_fuses(int count, const hipq_weight *const *w, int64_t M, const float *A, int64_t lda);
int launch_gemm_rows_q40_fused(int count, const hipq_weight *const *w, const float *A, int64_t lda, int M,
                               float *const *C, const int64_t *ldc, hipStream_t s);

/* moe.hip ----------------------------------------------------------------- */
/* Variant of the expert MLP. kind 0: h = silu(g) * u, y = down(h) (qwen_moe_layer.cpp:332-392).
 * kind 1: g and u take a bias, h = (g / (1 + exp(-alpha g))) * (u + 1), y = down(h) + bias
 * (gpt_oss_moe_layer.cpp:372-449); with limit > 0 the biased g and u are clamped first, g to
 * at most limit and u to [-limit, limit] (gpt_oss_moe_layer_cached.cpp:497-507). Biases are
 * device pointers, [E][I], [E][I], [E][H]. */
struct MoeEpi {
  const float *gate_bias, *up_bias, *down_bias;
  float alpha;
  float limit;
  int kind;
};
struct MoeArgs {
  hipq_moe_desc desc;
  MoeEpi epi;
  const float *router_bias; /* device [E] or null; applies to logits formed from router_weight */
  const hipq_weight *const *gate;
  const hipq_weight *const *up;
  const hipq_weight *const *down;
  const float *x;             /* device */
  const float *router_logits; /* device or null */
  const float *router_weight; /* device or null */
  float *y;                   /* device */
  int32_t *topk_idx;          /* device or null */
  float *topk_w;              /* device or null */
};
size_t moe_workspace_bytes(const hipq_moe_desc *d);
bool moe_wants_tiles(const hipq_moe_desc *d, int dtype); /* the block's experts run on the matrix cores */
int launch_moe(const MoeArgs *a, void *workspace, size_t workspace_bytes,
               const WView *dev_views /* [3*E] gate|up|down, device */,
               hipStream_t s);

/* wquant.hip -------------------------------------------------------------- */
int launch_quantize_weights(int dtype, const float *W, int64_t N, int64_t K,
                            void *out_blocks, hipStream_t s);

/* relayout.hip ------------------------------------------------------------ */
constexpr int EXPERT_TILE_BYTES = 4096 + 512; /* nibbles, then headers, of 32 rows and one super-block */
int tile_expert_weight(hipq_weight *w); /* planes -> 32-row tiles, in a new allocation; synchronous */
int ensure_gemm_tiles(hipq_weight *w);  /* adds the prefill GEMM's tile copy (allocates once; synchronous) */
int launch_relayout(hipq_weight *w, int layout, const uint8_t *src_dev,
                    hipStream_t s);

} // namespace hipq

/* ------------------------------------------------------------------------- */
/* device helpers                                                             */
/* ------------------------------------------------------------------------- */
#if defined(__HIPCC__)

#define HIPQ_WAVE 64

__device__ __forceinline__ float hipq_h2f(uint16_t bits) {
  return __half2float(__ushort_as_half(bits));
}
/* fp32 -> fp16, round to nearest even (F16C _cvtss_sh semantics). The sign is
 * copied from the fp32 bits: the compiler's conversion turns -0.0f into +0. */
__device__ __forceinline__ uint16_t hipq_f2h(float f) {
  const uint16_t h = __half_as_ushort(__float2half_rn(f));
  return (uint16_t)((h & 0x7fffu) | ((__float_as_uint(f) >> 16) & 0x8000u));
}

/* signed 4 x int8 dot product with int32 accumulate (v_dot4_i32_i8) */
__device__ __forceinline__ int hipq_dot4(int a, int b, int c) {
  return __builtin_amdgcn_sdot4(a, b, c, false);
}

template <int CTRL> __device__ __forceinline__ int hipq_dpp_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL> __device__ __forceinline__ float hipq_dpp_f(float v) {
  return __builtin_bit_cast(float, hipq_dpp_i<CTRL>(__builtin_bit_cast(int, v)));
}

/* DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror,
 * row_mirror. After the first four steps every lane of a 16-lane row holds the
 * row's total; rows are then combined with two cross-row exchanges. All lanes
 * of a group end with bit-identical values (each step adds the same two
 * operands in both partners). */
#define HIPQ_DPP_XOR1 0xB1
#define HIPQ_DPP_XOR2 0x4E
#define HIPQ_DPP_HALF_MIRROR 0x141
#define HIPQ_DPP_MIRROR 0x140

template <int T> __device__ __forceinline__ float hipq_group_sum(float v) {
  if (T >= 2) v += hipq_dpp_f<HIPQ_DPP_XOR1>(v);
  if (T >= 4) v += hipq_dpp_f<HIPQ_DPP_XOR2>(v);
  if (T >= 8) v += hipq_dpp_f<HIPQ_DPP_HALF_MIRROR>(v);
  if (T >= 16) v += hipq_dpp_f<HIPQ_DPP_MIRROR>(v);
  if (T >= 32) v += __shfl_xor(v, 16, HIPQ_WAVE);
  if (T >= 64) v += __shfl_xor(v, 32, HIPQ_WAVE);
  return v;
}
template <int T> __device__ __forceinline__ int hipq_group_sum_i(int v) {
  if (T >= 2) v += hipq_dpp_i<HIPQ_DPP_XOR1>(v);
  if (T >= 4) v += hipq_dpp_i<HIPQ_DPP_XOR2>(v);
  if (T >= 8) v += hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(v);
  if (T >= 16) v += hipq_dpp_i<HIPQ_DPP_MIRROR>(v);
  if (T >= 32) v += __shfl_xor(v, 16, HIPQ_WAVE);
  if (T >= 64) v += __shfl_xor(v, 32, HIPQ_WAVE);
  return v;
}
template <int T> __device__ __forceinline__ float hipq_group_max(float v) {
  if (T >= 2) v = fmaxf(v, hipq_dpp_f<HIPQ_DPP_XOR1>(v));
  if (T >= 4) v = fmaxf(v, hipq_dpp_f<HIPQ_DPP_XOR2>(v));
  if (T >= 8) v = fmaxf(v, hipq_dpp_f<HIPQ_DPP_HALF_MIRROR>(v));
  if (T >= 16) v = fmaxf(v, hipq_dpp_f<HIPQ_DPP_MIRROR>(v));
  if (T >= 32) v = fmaxf(v, __shfl_xor(v, 16, HIPQ_WAVE));
  if (T >= 64) v = fmaxf(v, __shfl_xor(v, 32, HIPQ_WAVE));
  return v;
}

/* The same reductions over the whole wavefront with a wave-uniform result, without the two
 * exchanges through the LDS crossbar that the last steps of the group forms take (about two hundred
 * clocks each when a lone wavefront waits for them): after the four steps inside the rows of sixteen
 * lanes, row_bcast:15 hands every row's value to the next row (rows 1 and 3 take it), row_bcast:31
 * hands row 1's to rows 2 and 3, and lane 63 holds the total, which a scalar read broadcasts. The
 * sum associates as the exchange form does, (R3 + R2) + (R1 + R0) over the rows' totals, so it has
 * that form's bits. */
template <int CTRL, int ROWS> __device__ __forceinline__ int hipq_dpp_rows_i(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, ROWS, 0xf, false); /* rows outside ROWS keep v */
}
__device__ __forceinline__ float hipq_wave_max(float v) {
  v = hipq_group_max<16>(v);
  v = fmaxf(v, __builtin_bit_cast(float, hipq_dpp_rows_i<0x142, 0xa>(__builtin_bit_cast(int, v))));
  v = fmaxf(v, __builtin_bit_cast(float, hipq_dpp_rows_i<0x143, 0xc>(__builtin_bit_cast(int, v))));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ int hipq_wave_min_i(int v) {
  v = min(v, hipq_dpp_i<HIPQ_DPP_XOR1>(v));
  v = min(v, hipq_dpp_i<HIPQ_DPP_XOR2>(v));
  v = min(v, hipq_dpp_i<HIPQ_DPP_HALF_MIRROR>(v));
  v = min(v, hipq_dpp_i<HIPQ_DPP_MIRROR>(v));
  v = min(v, hipq_dpp_rows_i<0x142, 0xa>(v));
  v = min(v, hipq_dpp_rows_i<0x143, 0xc>(v));
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ float hipq_wave_sum(float v) {
  v = hipq_group_sum<16>(v);
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xa, 0xf, false));
  v = v + r1; /* rows 0 and 2 add zero */
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xc, 0xf, false));
  v = v + r2;
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

/* Inclusive prefix sum over the lanes of a wavefront by shifted adds inside the rows of sixteen
 * lanes (row_shr 1, 2, 4, 8: lanes without a source add zero) and the two row-broadcast steps. */
__device__ __forceinline__ int hipq_wave_prefix_sum_i(int v) {
  v += hipq_dpp_i<0x111>(v);
  v += hipq_dpp_i<0x112>(v);
  v += hipq_dpp_i<0x114>(v);
  v += hipq_dpp_i<0x118>(v);
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false); /* rows 1 and 3 take the total of the row before */
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false); /* rows 2 and 3 take the total of rows 0 and 1 */
  return v;
}

/* Loads of weight data name the global address space. A pointer that a kernel
 * read from memory (a table of weight views) is generic to the compiler, which
 * then emits flat loads; those count against the LDS counter as well, so every
 * wait for an LDS read would also wait for the weight prefetch. */
#define HIPQ_GLOBAL __attribute__((address_space(1)))
typedef unsigned int hipq_u32x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ T hipq_ld_global(const T *p) {
  if constexpr (sizeof(T) == 16) {
    return __builtin_bit_cast(T, *(const HIPQ_GLOBAL hipq_u32x4 *)p);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, *(const HIPQ_GLOBAL uint32_t *)p);
  } else {
    static_assert(sizeof(T) == 2, "16-, 4- and 2-byte loads only");
    return __builtin_bit_cast(T, *(const HIPQ_GLOBAL uint16_t *)p);
  }
}
/* 128-bit streaming load of weight data: marked non-temporal so the one-pass
 * weight stream does not evict the (re-used) quantized activations. */
__device__ __forceinline__ uint4 hipq_ld_stream(const uint4 *p) {
  hipq_u32x4 v = __builtin_nontemporal_load((const HIPQ_GLOBAL hipq_u32x4 *)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

#endif /* __HIPCC__ */
#endif /* HIPQ_INTERNAL_H */
