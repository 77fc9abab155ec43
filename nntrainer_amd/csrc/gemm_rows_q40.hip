// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm_rows_q40.hip
 * @brief  Q4_0 x Q8_0 for a few activation rows (two to 64, in passes of eight side by side
 *         in one launch) on the int8 matrix cores, with the reference's bits.
 *
 * Replaces what __ggml_q4_0_8x8_q8_0_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:303-389 in the
 * reference checkout) does with a few rows through nntr_gemv_q4_0_8x8_q8_0 and
 * nntr_gemm_q4_0_8x8_q8_0 (nntr_ggml_impl.cpp:650-3259): per output one fp32 sum,
 * acc = fma(float(sum of the block's 32 integer products), d_w * d_a, acc), block after block.
 * Both of the reference's kernels order it that way, so rows are independent of each other.
 * The GEMV engine (gemv_device.h) forms the integer sums on the vector ALU, where every further
 * row costs about as much as the first; the prefill GEMM (gemm.hip) works on tiles of 64 rows.
 *
 * Here a workgroup owns 32 output columns and the eight rows of its pass (blockIdx.y). A round
 * is 32 blocks of K; each of the four wavefronts takes eight of them: one
 * v_mfma_i32_32x32x32_i8 per block (the activation rows are the row operand: 8 of its 32 rows
 * are used) on the nibbles as they are (0..15), whose exact int32 sums go to LDS; after a
 * barrier every thread runs the fp32 chain of ONE output over the round's blocks in ascending
 * order, taking 8 * (sum of the block's activations) off each sum first (the quantizer stores
 * that sum beside the scale), so the chain is as long as on the vector ALU but the integer work
 * is not. The eight blocks of a column and round are one 128-byte line: a load instruction
 * fetches eight whole lines, which reach the lanes of their columns through LDS, and the two
 * lanes of a column swap nibble halves with v_permlane32_swap; the loads of the next round are
 * in flight during the current one and are
 * issued unconditionally (past the end the last blocks again: behind a condition the compiler
 * cannot count the loads in flight and waits for all of them). Activations, their scales and
 * the weights' scales are staged a round at a time (46 KB of LDS with the sums: three
 * workgroups a CU, any K).
 */
#include "hipq_internal.h"
#include "gemv_device.h"
#include "quantize_device.h"

namespace {

typedef int qv2i __attribute__((ext_vector_type(2)));
typedef int qv4i __attribute__((ext_vector_type(4)));
typedef float qv4f __attribute__((ext_vector_type(4)));
typedef int qv16i __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t qrsrc_t;

constexpr int TC = 8;        /* activation rows a workgroup holds */
constexpr int NREG = 4;      /* result registers of a matrix step that carry them */
constexpr int WV = 4;        /* wavefronts a workgroup */
constexpr int BW = 8;        /* blocks a wavefront takes per round */
constexpr int BR = WV * BW;  /* blocks a round */
constexpr int NT = 64 * WV;

/* LDS of a workgroup.
 *   q    [row][BR * 32 + 32]: the int8 values of the round's blocks (rows padded so that the
 *        sixteen 16-byte pieces a matrix step reads fall into different banks); written behind
 *        a round's first barrier for the next round, when nobody reads it any more
 *   da   [row][BR] fp32 scales, s8 [row][BR] eight times the block sums: written at the start of
 *        the round that uses them (the chains of the round before are done), read by the chains
 *   dw   [four blocks][column][4] fp32 scales of the weights, likewise
 *   rec  [wavefront][blocks 0-3 | 4-7][register][lane][4]: the sums of a round, so that a lane
 *        writes, and a chain reads, four blocks as one 128-bit access */
constexpr int QROW = BR * 32 + 32;
constexpr int LDS_Q = 0;
constexpr int LDS_DA = LDS_Q + TC * QROW;
constexpr int LDS_S8 = LDS_DA + TC * BR * 4;
constexpr int LDS_DW = LDS_S8 + TC * BR * 4;
constexpr int LDS_REC = LDS_DW + 32 * BR * 4;
constexpr int REC_DWORDS = WV * 2 * NREG * 64 * 4;
constexpr int SROW = 128 + 16; /* a column's line in the staging, padded against bank conflicts */
static_assert(32 * SROW <= 2 * NREG * 256 * 4, "the staged lines fit a wavefront's records");
constexpr int LDS_BYTES = LDS_REC + REC_DWORDS * 4;
static_assert(LDS_REC % 16 == 0 && 3 * LDS_BYTES <= 160 * 1024, "three workgroups a CU");

struct WRegs {
  qv4i x[4]; /* load i: block lane % 8 of the wavefront's eight, column 8 i + lane / 8 */
};

/* what a thread stages per round besides the int8 values: the metadata word of one (row, block)
 * and four fp16 scales of one column */
struct SRegs {
  uint32_t meta;
  uint2 dw;
};

/* Up to four weights of one K against the same quantized rows as ONE launch: the grid's columns are
 * the concatenation of the weights' column tiles (Q, K, V or gate, up of a layer). */
struct MultiRowsQ40 {
  WView w[4];
  float *C[4];
  int64_t ldc[4];
  int tile_end[4]; /* running sum of the weights' column tiles */
};

/* FUSED: the rows come as fp32 (Af, row stride lda) and every workgroup quantizes its pass's rows
 * itself, a round ahead, with the arithmetic of the Q8_0 quantizer kernel (the same bits): no
 * quantizer launch and no workspace. For launches of few workgroups, where that launch costs more
 * than the repeated quantization. */
template <bool FUSED>
__global__ __launch_bounds__(NT, 2) void gemm_rows_q40_kernel(MultiRowsQ40 mw, QView a, const float *__restrict__ Af,
                                                              int64_t lda, int M_all) {
  extern __shared__ __attribute__((aligned(16))) unsigned char rows_lds[];
  /* which weight this workgroup's column tile belongs to (uniform) */
  int tile = blockIdx.x, wi = 0;
  if (tile >= mw.tile_end[0]) wi = 1;
  if (tile >= mw.tile_end[1]) wi = 2;
  if (tile >= mw.tile_end[2]) wi = 3;
  if (wi) tile -= mw.tile_end[wi - 1];
  const WView w = wi == 0 ? mw.w[0] : wi == 1 ? mw.w[1] : wi == 2 ? mw.w[2] : mw.w[3];
  float *__restrict__ C = wi == 0 ? mw.C[0] : wi == 1 ? mw.C[1] : wi == 2 ? mw.C[2] : mw.C[3];
  const int64_t ldc = wi == 0 ? mw.ldc[0] : wi == 1 ? mw.ldc[1] : wi == 2 ? mw.ldc[2] : mw.ldc[3];
  const int K = w.K, nb = K >> 5;
  const int r0 = blockIdx.y * TC;
  const int M = min(TC, M_all - r0);
  if (FUSED) {
    Af += (int64_t)r0 * lda;
  } else {
    a.q += (size_t)r0 * K;
    a.meta += (size_t)r0 * nb;
  }
  C += (int64_t)r0 * ldc;
  const int n0 = tile * 32;
  const int ncols = min(32, w.N - n0);
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63, i32 = lane & 31, g = lane >> 5;
  const int t = threadIdx.x;
  uint32_t *const lrec = (uint32_t *)(rows_lds + LDS_REC);

  /* the tile's nibbles as a buffer descriptor in scalar registers; columns past N repeat the last */
  const qrsrc_t rq = __builtin_amdgcn_make_buffer_rsrc((void *)(w.qs + (size_t)n0 * (size_t)(K >> 1)), 0,
                                                       ncols * (K >> 1), 0x00020000);
  /* load i of a lane: 16 bytes of column 8 i + lane / 8, so that eight lanes cover the 128-byte line a
   * column's eight blocks are and a load instruction eight whole lines (a lane loading its own
   * column's blocks touches 32 lines for 32 bytes of each: 14.3 against 10.5 us at 12288 x 4096) */
  int wvoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) wvoff[i] = min(8 * i + (lane >> 3), ncols - 1) * (K >> 1) + (lane & 7) * 16;
  auto load = [&](WRegs &r, int rho) {
    const int b0 = min(rho * BR + wave * BW, nb - BW); /* uniform; a wavefront past the end loads the last blocks and does not use them */
#pragma unroll
    for (int i = 0; i < 4; ++i)
      r.x[i] = __builtin_bit_cast(qv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, wvoff[i], b0 * 16, 2));
  };
  /* Rows M .. TC - 1 repeat row M - 1 and pieces past the end of a row its last piece: every
   * thread always issues the same loads, and what they fetch there is never used. */
  auto q_load = [&](qv4i (&r)[2], int rho) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = t + u * NT;
      const int row = min(c >> 6, M - 1), off = min(rho * (BR * 32) + (c & 63) * 16, K - 16);
      r[u] = *(const qv4i *)(a.q + (size_t)row * K + off);
    }
  };
  auto q_store = [&](const qv4i (&r)[2]) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = t + u * NT;
      *(qv4i *)(rows_lds + LDS_Q + (c >> 6) * QROW + (c & 63) * 16) = r[u];
    }
  };
  const uint16_t *const dcol = w.d + (size_t)(n0 + min(t >> 3, ncols - 1)) * nb;
  auto s_load = [&](SRegs &r, int rho) {
    if (!FUSED) r.meta = a.meta[(size_t)min(t >> 5, M - 1) * nb + min(rho * BR + (t & 31), nb - 1)];
    r.dw = *(const uint2 *)(dcol + min(rho * BR + (t & 7) * 4, nb - 4));
  };
  auto s_store = [&](const SRegs &r) {
    ((float *)(rows_lds + LDS_DA))[t] = hipq_h2f((uint16_t)(r.meta & 0xffff)); /* [row][block] */
    ((int *)(rows_lds + LDS_S8))[t] = ((int)r.meta >> 16) * 8;
    const qv4f f = {hipq_h2f((uint16_t)(r.dw.x & 0xffff)), hipq_h2f((uint16_t)(r.dw.x >> 16)),
                    hipq_h2f((uint16_t)(r.dw.y & 0xffff)), hipq_h2f((uint16_t)(r.dw.y >> 16))};
    *(qv4f *)(rows_lds + LDS_DW + ((t & 7) * 32 + (t >> 3)) * 16) = f; /* [four blocks][column][4] */
  };

  /* FUSED: a thread takes one block of a round, row t / 32, block t % 32: 32 fp32 values in, its 32
   * int8 values to LDS, the block's metadata word (fp16 scale, sum of the values) back */
  struct FRegs {
    float4 x[FUSED ? 8 : 1];
  };
  auto f_load = [&](FRegs &r, int rho) {
    const float4 *p = (const float4 *)(Af + (int64_t)min(t >> 5, M - 1) * lda + min(rho * (BR * 32) + (t & 31) * 32, K - 32));
#pragma unroll
    for (int i = 0; i < 8; ++i) r.x[i] = p[i];
  };
  auto f_quant_store = [&](const FRegs &r) -> uint32_t {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      amax = fmaxf(amax, fmaxf(fmaxf(fabsf(r.x[i].x), fabsf(r.x[i].y)), fmaxf(fabsf(r.x[i].z), fabsf(r.x[i].w))));
    const float d = __fdiv_rn(amax, 127.f);
    const float id = (amax != 0.0f) ? __fdiv_rn(127.f, amax) : 0.0f;
    int pk[8], sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q0 = (int)rintf(__fmul_rn(r.x[i].x, id)), q1 = (int)rintf(__fmul_rn(r.x[i].y, id));
      const int q2 = (int)rintf(__fmul_rn(r.x[i].z, id)), q3 = (int)rintf(__fmul_rn(r.x[i].w, id));
      pk[i] = pack4(q0, q1, q2, q3);
      sum += (q0 + q1) + (q2 + q3);
    }
    unsigned char *dst = rows_lds + LDS_Q + (t >> 5) * QROW + (t & 31) * 32;
    *(qv4i *)dst = qv4i{pk[0], pk[1], pk[2], pk[3]};
    *(qv4i *)(dst + 16) = qv4i{pk[4], pk[5], pk[6], pk[7]};
    return (uint32_t)hipq_f2h(d) | ((uint32_t)(sum & 0xffff) << 16);
  };

  constexpr int PD = 1, NB = PD + 1;
  WRegs buf[NB];
  qv4i AQ[2];
  FRegs FR;
  SRegs SR;
  const int rounds = (nb + BR - 1) / BR;
  if (FUSED) f_load(FR, 0); else q_load(AQ, 0);
  s_load(SR, 0);
#pragma unroll
  for (int p = 0; p < PD; ++p) load(buf[p], p);
  if (FUSED) SR.meta = f_quant_store(FR); else q_store(AQ);
  __syncthreads();

  /* the output this thread chains: row cm, column cn; its sums sit in register cr of lane cl */
  const int cn = t & 31, cm = t >> 5;
  const int cr = cm & 3, cl = (cm >> 2) * 32 + cn;
  float acc = 0.f;
  const bool chains = 2 * wave < M; /* uniform: a wavefront chains rows 2 wave and 2 wave + 1 */

  auto round = [&](const WRegs &W, int rho) {
    if (rho * BR + wave * BW < nb) { /* uniform per wavefront */
      const qv16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const int8_t *pa = (const int8_t *)rows_lds + LDS_Q + (i32 & (TC - 1)) * QROW + wave * (BW * 32) + g * 16;
      qv4i a8[BW];
#pragma unroll
      for (int j = 0; j < BW; ++j) a8[j] = *(const qv4i *)(pa + j * 32);
      /* the loaded lines go through the wavefront's own part of the records (free until its sums are
       * written; LDS serves a wavefront's accesses in order) to the lanes of their columns: lane
       * (n, g) takes blocks 2 i + g of column n */
      unsigned char *stage = (unsigned char *)(lrec + wave * (2 * NREG * 256));
#pragma unroll
      for (int i = 0; i < 4; ++i) *(qv4i *)(stage + (8 * i + (lane >> 3)) * SROW + (lane & 7) * 16) = W.x[i];
      __builtin_amdgcn_wave_barrier();
      qv4i X[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) X[i] = *(const qv4i *)(stage + i32 * SROW + (2 * i + g) * 16);
      /* wq[j]: this lane's half of block j, one nibble a byte: the low nibbles (values 0..15 of the
       * block) in the lanes of g = 0, the high ones (16..31) in those of g = 1 */
      qv4i wq[BW];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t x = (uint32_t)X[i][d];
          const auto s = __builtin_amdgcn_permlane32_swap(x & HIPQ_M4, (x >> 4) & HIPQ_M4, false, false);
          wq[2 * i][d] = (int)s[0];
          wq[2 * i + 1][d] = (int)s[1];
        }
      }
      uint32_t *rec = lrec + wave * (2 * NREG * 256) + lane * 4;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        qv16i D[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) D[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8[4 * h + j], wq[4 * h + j], zero16, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < NREG; ++r)
          *(qv4i *)(rec + (h * NREG + r) * 256) = qv4i{D[0][r], D[1][r], D[2][r], D[3][r]};
      }
    }
    __syncthreads();
    /* the next round's values: nobody reads this round's any more */
    if (FUSED) SR.meta = f_quant_store(FR); else q_store(AQ);
    /* the chains of this round's blocks, ascending (the records of a wavefront that had no blocks
     * are read as well and not used: a read behind a branch would wait for its own latency) */
    const float *lda_ = (const float *)(rows_lds + LDS_DA) + cm * BR;
    const int *ls8 = (const int *)(rows_lds + LDS_S8) + cm * BR;
    const float *ldw = (const float *)(rows_lds + LDS_DW) + cn * 4;
    if (chains) {
#pragma unroll
    for (int ws = 0; ws < WV; ++ws) {
      qv4i dv[2], sv[2];
      qv4f av[2], wv[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        dv[h] = *(const qv4i *)(lrec + ws * (2 * NREG * 256) + (h * NREG + cr) * 256 + cl * 4);
        sv[h] = *(const qv4i *)(ls8 + ws * BW + h * 4);
        av[h] = *(const qv4f *)(lda_ + ws * BW + h * 4);
        wv[h] = *(const qv4f *)(ldw + (ws * 2 + h) * 128);
      }
      if (rho * BR + ws * BW < nb) { /* uniform */
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = fmaf((float)(dv[h][j] - sv[h][j]), av[h][j] * wv[h][j], acc);
      }
    }
    }
    __syncthreads(); /* the next round overwrites the records and the scales */
  };
  /* NB rounds a trip so that each register set has a fixed name; all conditions are uniform */
  for (int rho0 = 0; rho0 < rounds; rho0 += NB) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int rho = rho0 + u;
      if (rho < rounds) {
        s_store(SR); /* this round's scales: the chains of the round before have passed their barrier */
        /* before the weights: their waits must not include the weights' */
        if (FUSED) f_load(FR, rho + 1); else q_load(AQ, rho + 1);
        s_load(SR, rho + 1);
        load(buf[(u + PD) % NB], rho + PD);
        round(buf[u], rho);
      }
    }
  }
  const int col = n0 + cn;
  if (cm < M && col < w.N) C[(int64_t)cm * ldc + col] = acc;
}

} // namespace

namespace hipq {

/* Where it beats what served these row counts before (measured, whole call with the quantizer, us
 * old -> new). The GEMV engine, a row at a time in effect: 12288 x 4096 with 2 / 4 / 8 rows 13.5 /
 * 15.2 / 28.3 -> 12.9 / 12.9 / 13.4; 151936 x 1024 42.7 / 54.7 / 68.0 -> 26.5 / 27.2 / 28.8 (one row:
 * 31.7 -> 26.0; with K = 2048 and more one row stays with the engine: 37.6 against 42.3); 4096 x 4096
 * 8.8 / 9.5 / 15.0 -> 9.9 / 10.5 / 10.8; 3072 x 1024 5.4 / 5.9 / 8.0 -> 6.4 / 6.8 / 7.0; 1024 x 3072
 * with 8 rows 7.7 against 9.4. The prefill GEMM, one 64-row tile whatever the row count: 16 rows at
 * 12288 x 4096 28.3 -> 17.6, 4096 x 4096 19.4 -> 10.9, 1024 x 3072 15.1 -> 9.4, 1024 x 1024 8.5 -> 6.7,
 * 151936 x 1024 68.4 -> 49.0; with more passes the launch grows and the GEMM does not: 12288 x 4096
 * with 24 / 32 rows 25.2 / 29.6 against 28.4 / 28.5, 4096 x 4096 with 48 / 64 rows 16.5 / 20.3 against
 * 19.7 / 19.9, 151936 x 1024 with 24 rows 71.7 against 68.7, 1024 x 3072 with 64 rows 9.5 against 15.4.
 * Against the engine with its row lengths compiled in (calls in a row on one stream, us, engine
 * against this kernel): two rows 12288 x 4096 12.2 / 13.1, 12288 x 2048 9.2 / 9.6, 32768 x 4096 22.0 /
 * 21.6, 65536 x 2048 24.9 / 22.8, 151936 x 2048 49.2 / 43.0; three and four rows 6144 x 4096 10.5 / 10.8,
 * 12288 x 4096 14.3 / 13.2, 4096 x 2048 7.1 / 7.7, 12288 x 2048 10.9 / 9.6. Where the kernel quantizes
 * the rows itself (K of one round, up to 512 tiles) it is one launch against the engine's two, and
 * two to eight rows take it from 512 columns: 512 ... 3072 x 1024 with two to four 7.0 / 5.3, 6144 x
 * 1024 7.1 / 5.5, 3072 x 1024 with six and eight 8.0 / 5.5. */
static bool rows_q40_pay(int64_t N, int64_t K, int64_t M) {
  if (M == 1) return false; /* the streamed GEMV, since its waits count every load: 151936 x 1024 28.5 -> 18.3 us a call, 65536 x 1024 15.2 -> 10.6 */
  const bool quantizes = K <= BR * 32 && (N + 31) / 32 <= 512; /* one launch: the form that takes the fp32 rows */
  if (M <= TC && quantizes) return N >= 512;
  if (M == 2) return N >= (K <= BR * 32 ? 12288 : 32768);
  if (M <= 4) return N >= 6144;
  if (M <= TC) return N >= 3072;
  if (M <= 2 * TC) return N >= 512;
  if (M > 8 * TC || N < 512) return false;
  const int64_t tiles = (N + 31) / 32, passes = (M + TC - 1) / TC, rounds = (K / 32 + BR - 1) / BR;
  return tiles * passes * (rounds + 1) <= 6000;
}

static bool rows_q40_can(const hipq_weight *w) {
  return w->dtype == HIPQ_Q4_0 && w->K % 256 == 0 && 16 * w->K <= 0x7fffffff;
}

bool gemm_rows_q40_fits(const hipq_weight *w, int64_t M) { return rows_q40_can(w) && rows_q40_pay(w->N, w->K, M); }

/* Several weights of one K in one launch: what counts is the launch's width, the columns of all of
 * them, and the launches it replaces. The seven FCs of a Qwen3-0.6B-shaped decoder layer with Q, K, V
 * and gate, up as one call each, replayed from a graph, us per layer with 2 / 4 / 8 / 16 / 32 rows:
 * 31.4 / 35.3 / 37.1 / 34.9 / 35.0 with a launch per weight (or the prefill GEMM's grouped launch from
 * nine rows) -> 23.2 / 25.4 / 26.4 / 29.8 / 32.4. */
bool gemm_rows_q40_fits_multi(int count, const hipq_weight *const *w, int64_t M) {
  if (count < 1 || count > 4) return false;
  int64_t N = 0;
  for (int i = 0; i < count; ++i) {
    if (!rows_q40_can(w[i]) || w[i]->K != w[0]->K) return false;
    N += (w[i]->N + 31) / 32 * 32;
  }
  if (count == 1) return rows_q40_pay(N, w[0]->K, M);
  if (M < 2 || M > 8 * TC || N < 1024) return false;
  if (M <= 2 * TC) return true;
  const int64_t tiles = N / 32, passes = (M + TC - 1) / TC, rounds = (w[0]->K / 32 + BR - 1) / BR;
  return tiles * passes * (rounds + 1) <= 6000;
}

/* qa: the quantized rows, or null with the fp32 rows A (row stride lda) for the form that quantizes them itself */
static int launch_rows_q40(int count, const hipq_weight *const *w, const QAct *qa, const float *A, int64_t lda, int M,
                           float *const *C, const int64_t *ldc, hipStream_t s) {
  if (count < 1 || count > 4) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_0 product takes 1 to 4 weights a launch");
  if (M < 1 || M > 8 * TC) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_0 product takes 1..64 rows");
  MultiRowsQ40 mw;
  int tiles = 0;
  for (int i = 0; i < 4; ++i) {
    const int j = i < count ? i : count - 1;
    if (i < count) {
      if (!rows_q40_can(w[i]) || w[i]->K != (qa ? qa->K : w[0]->K))
        return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_0 product takes Q4_0 weights of the rows' K, in whole 256s");
      tiles += (int)((w[i]->N + 31) / 32);
    }
    mw.w[i] = wview(w[j]);
    mw.C[i] = C[j];
    mw.ldc[i] = ldc[j];
    mw.tile_end[i] = tiles; /* unused entries repeat the total: no workgroup lands in them */
  }
  const dim3 grid((unsigned)tiles, (unsigned)((M + TC - 1) / TC));
  if (qa) {
    hipq::launch_kernel("gemm_rows_q40_kernel<false>", gemm_rows_q40_kernel<false>, grid, dim3(NT), LDS_BYTES, s, mw, qview(*qa), (const float *)nullptr,
                       (int64_t)0, M);
  } else {
    QView none{};
    none.K = (int)w[0]->K;
    hipq::launch_kernel("gemm_rows_q40_kernel<true>", gemm_rows_q40_kernel<true>, grid, dim3(NT), LDS_BYTES, s, mw, none, A, lda, M);
  }
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_gemm_rows_q40_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, float *const *C,
                               const int64_t *ldc, hipStream_t s) {
  return launch_rows_q40(count, w, qa, nullptr, 0, M, C, ldc, s);
}

/* The form that quantizes the fp32 rows itself: where the launch would take the few-rows kernel
 * anyway, is small, and K is one round: the kernel then starts a microsecond later (fp32 rows in,
 * quantized, a barrier before the first matrix step) and saves a quantizer launch of 2.5 us.
 * Whole calls, us, two launches -> one: 3072 x 1024 with 8 rows 7.0 -> 5.7, 2048 x 1024 with 16 rows
 * 6.7 -> 5.5, 1024 x 1024 6.7 -> 5.6; with three rounds it loses (1024 x 3072 with 16 rows 9.4 ->
 * 10.1), with two it gains nothing (512 x 2048 7.7 -> 7.8). */
bool gemm_rows_q40_fuses(int count, const hipq_weight *const *w, int64_t M, const float *A, int64_t lda) {
  if (!gemm_rows_q40_fits_multi(count, w, M) || ((uintptr_t)A & 15) || (lda & 3)) return false;
  int64_t tiles = 0;
  for (int i = 0; i < count; ++i) tiles += (w[i]->N + 31) / 32;
  return w[0]->K <= BR * 32 && tiles <= 512;
}

int launch_gemm_rows_q40_fused(int count, const hipq_weight *const *w, const float *A, int64_t lda, int M,
                               float *const *C, const int64_t *ldc, hipStream_t s) {
  if (((uintptr_t)A & 15) || (lda & 3)) return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  return launch_rows_q40(count, w, nullptr, A, lda, M, C, ldc, s);
}

int launch_gemm_rows_q40(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  return launch_gemm_rows_q40_multi(1, &w, qa, M, &C, &ldc, s);
}

} // namespace hipq
