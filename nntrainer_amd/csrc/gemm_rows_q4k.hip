// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm_rows_q4k.hip
 * @brief  Q4_K x Q8_K for a few activation rows (three to 64, in passes of eight side by
 *         side in one launch) on the int8 matrix cores, with the reference's bits.
 *
 * Replaces, for 3 <= M <= 64, what __ggml_q4_K_8x8_q8_K_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:391-517 in the
 * reference checkout) does with a few rows: the rows below 4 * (M / 4) go through
 * nntr_gemm_q4_K_8x8_q8_K (nntr_ggml_impl.cpp:3261-7078), which adds the four sub-block
 * pairs of a super-block to a row's sum one after the other, the others through
 * nntr_gemv_q4_K_8x8_q8_K (:7080-7494), which adds the super-block's total. The GEMV engine
 * (gemv_device.h) does the same on the vector ALU, where a row of activations costs about
 * 4 us on a 12288 x 4096 matrix (eight rows: 37 us; one row: 8 us, the weight stream); this
 * kernel takes 11.2 us for eight.
 *
 * Here a workgroup owns 32 output columns and the eight rows of its pass (blockIdx.y). Its four wavefronts take one
 * super-block each per round: one v_mfma_i32_32x32x32_i8 per sub-block (the rows are the
 * row operand: 8 of its 32 rows are used), the 6-bit scales applied to the exact int32 sums
 * pair by pair, the mins through four v_mfma_f32_32x32x16_f16 with all but one pair's mins
 * zeroed. The four partial sums of both kinds go to LDS as they are (integers), and after a
 * barrier every thread runs the fp32 chain of ONE output over the round's super-blocks in
 * ascending order, exactly as the reference orders it, so the chain is as long as on the
 * vector ALU but the integer work is not. Weights come from the 32-row tile copy the prefill
 * GEMM reads (piece i of lane (n, g) = sub-block 4 g + i of row n; the two lanes of a row swap
 * halves with v_permlane32_swap so that each holds its 16 weights of sub-blocks i and 4 + i),
 * the loads of the next round in flight during the current one. The quantized rows are
 * staged a round at a time (52 KB of LDS with the records: three workgroups a CU, any K).
 */
#include "hipq_internal.h"
#include "gemv_device.h"

namespace {

typedef int rv2i __attribute__((ext_vector_type(2)));
typedef int rv4i __attribute__((ext_vector_type(4)));
typedef int rv16i __attribute__((ext_vector_type(16)));
typedef float rv16f __attribute__((ext_vector_type(16)));
typedef _Float16 rv8h __attribute__((ext_vector_type(8)));
typedef __amdgpu_buffer_rsrc_t rrsrc_t;

constexpr int TC = 8;    /* activation rows a workgroup holds */
constexpr int NREG = 4;  /* result registers of a matrix step that carry them */
constexpr int SBR = 4;   /* super-blocks a round = wavefronts a workgroup */
constexpr int NT = 64 * SBR;
/* a round's partial sums: [wavefront][register][integer sums | min sums][lane][pair 0-3], so that a
 * lane writes, and a chain reads, the four pairs of one kind as one 128-bit access, consecutive
 * lanes consecutive in memory */
constexpr int REC_DWORDS = SBR * NREG * 2 * 64 * 4;

/* LDS of a workgroup: the quantized rows of the current and of the next round (four
 * super-blocks of every row: int8 values, the sub-block sums as two fp16-exact parts, the
 * scales), the round's partial sums, and d and dmin of its super-blocks per column. */
constexpr int QROW = SBR * 256 + 16; /* a staged row, padded so that the lanes of a 128-bit read fall into different banks */
constexpr int ACT_Q = 0, ACT_AMIN = TC * QROW, ACT_DA = ACT_AMIN + TC * SBR * 32;
constexpr int ACT_BYTES = ACT_DA + SBR * TC * 4;
constexpr int LDS_REC = (2 * ACT_BYTES + 255) / 256 * 256;
constexpr int LDS_DW = LDS_REC + REC_DWORDS * 4;
constexpr int LDS_BYTES = LDS_DW + SBR * 2 * 32 * 4;
static_assert(ACT_BYTES % 16 == 0 && 3 * LDS_BYTES <= 160 * 1024, "three workgroups a CU");

struct RowsRegs {
  rv4i q[4];
  rv4i hd;
};

/* Up to four weights of one K against the same quantized rows as ONE launch: the grid's columns are
 * the concatenation of the weights' column tiles (Q, K, V or gate, up of a layer). */
struct MultiRowsQ4K {
  WView w[4]; /* qs, hdr: the tile copy */
  float *C[4];
  int64_t ldc[4];
  int tile_end[4]; /* running sum of the weights' column tiles */
};

/* blockIdx.y: the pass, rows 8 y .. 8 y + 7 of the call's M_all (the first pair_all of them under
 * the 4-row rule); the passes of one launch run side by side */
__global__ __launch_bounds__(NT, 2) void gemm_rows_q4k_kernel(MultiRowsQ4K mw, QView a, int M_all, int pair_all) {
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
  const int K = w.K, nsb = K >> 8;
  const int r0 = blockIdx.y * TC;
  const int M = min(TC, M_all - r0), pair_rows = min(max(pair_all - r0, 0), M);
  a.q += (size_t)r0 * K;
  a.d += (size_t)r0 * nsb;
  a.bsum += (size_t)r0 * (K >> 4);
  C += (int64_t)r0 * ldc;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63, i32 = lane & 31, g = lane >> 5;
  uint32_t *const lrec = (uint32_t *)(rows_lds + LDS_REC);
  float *const ldw = (float *)(rows_lds + LDS_DW);

  /* the tile's nibbles and headers as buffer descriptors in scalar registers */
  const rrsrc_t rq = __builtin_amdgcn_make_buffer_rsrc((void *)(w.qs + (size_t)tile * (size_t)(16 * K)), 0, 16 * K, 0x00020000);
  const rrsrc_t rh = __builtin_amdgcn_make_buffer_rsrc((void *)(w.hdr + (size_t)tile * (size_t)(nsb * 512)), 0, nsb * 512, 0x00020000);
  auto load = [&](RowsRegs &r, int sb) {
    sb = min(sb, nsb - 1); /* uniform; a wavefront past the end loads the last super-block and does not use it */
#pragma unroll
    for (int i = 0; i < 4; ++i)
      r.q[i] = __builtin_bit_cast(rv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, lane * 16, sb * 4096 + i * 1024, 2));
    r.hd = __builtin_bit_cast(rv4i, __builtin_amdgcn_raw_buffer_load_b128(rh, i32 * 16, sb * 512, 0));
  };
  /* A round's share of the M quantized rows goes through registers into one of two LDS buffers:
   * loaded (from the cache) at the start of the previous round, stored behind that round's first
   * barrier. Rows M .. TC - 1 repeat row M - 1 and pieces past the end of a row its last piece:
   * every thread always issues the same loads, and what they fetch there is never used. */
  struct ActRegs {
    rv4i q[2], amin;
    float dA;
  };
  auto act_load = [&](ActRegs &r, int rho) {
    const int t = threadIdx.x;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = t + u * NT;
      const int row = min(c >> 6, M - 1), off = min(rho * (SBR * 256) + (c & 63) * 16, K - 16);
      r.q[u] = *(const rv4i *)(a.q + (size_t)row * K + off);
    }
    {
      const int tt = t & 63, row = min(tt >> 3, M - 1);
      const int off = min(rho * (SBR * 32) + (tt & 7) * 16, nsb * 32 - 16);
      r.amin = *(const rv4i *)((const uint8_t *)a.bsum + (size_t)row * nsb * 32 + off);
    }
    {
      const int tt = t & 31, row = min(tt >> 2, M - 1);
      r.dA = a.d[(size_t)row * nsb + min(rho * SBR + (tt & 3), nsb - 1)];
    }
  };
  auto act_store = [&](const ActRegs &r, int which) {
    unsigned char *base = rows_lds + which * ACT_BYTES;
    const int t = threadIdx.x;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = t + u * NT;
      *(rv4i *)(base + ACT_Q + (c >> 6) * QROW + (c & 63) * 16) = r.q[u];
    }
    if (t < 64) *(rv4i *)(base + ACT_AMIN + t * 16) = r.amin; /* [row][super-block of the round][32 bytes] */
    if (t < 32) ((float *)(base + ACT_DA))[(t & 3) * TC + (t >> 2)] = r.dA; /* [super-block][row] */
  };
  ActRegs AR;
  act_load(AR, 0);
  /* The weights of PD + 1 rounds: the loads of the next PD rounds are in flight during a round.
   * Every round issues its loads, past the end those of the last super-block again: with a
   * conditional load the compiler cannot count the loads in flight and waits for all of them.
   * One round ahead keeps the kernel at 162 VGPRs, three wavefronts a SIMD as the LDS allows;
   * two rounds ahead (182) cost a third of them: 151936 x 4096 with eight rows 91 against 75 us. */
  constexpr int PD = 1, NB = PD + 1;
  RowsRegs buf[NB];
  const int rounds = (nsb + SBR - 1) / SBR;
#pragma unroll
  for (int p = 0; p < PD; ++p) load(buf[p], p * SBR + wave);
  act_store(AR, 0);
  __syncthreads();

  /* the output this thread chains: row cm, column cn; its sums sit in register cr of lane cl */
  const int cn = threadIdx.x & 31, cm = threadIdx.x >> 5;
  const int cr = cm & 3, cl = (cm >> 2) * 32 + cn;
  const bool pairwise = cm < pair_rows;
  float acc = 0.f, accm = 0.f;

  auto round = [&](const RowsRegs &W, int rho) {
    const unsigned char *act = rows_lds + (rho & 1) * ACT_BYTES;
    const int sb = rho * SBR + wave;
    if (sb < nsb) { /* uniform per wavefront */
      const rv16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const rv16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const int row = i32 & (TC - 1);
      const int8_t *pa = (const int8_t *)act + ACT_Q + row * QROW + wave * 256 + g * 16;
      const rv8h amin = *(const rv8h *)(act + ACT_AMIN + (row * SBR + wave) * 32 + g * 16);
      /* wq[j]: this lane's 16 weights (8 bytes) of sub-block j */
      rv2i wq[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const auto r0 = __builtin_amdgcn_permlane32_swap((unsigned)W.q[i][0], (unsigned)W.q[i][2], false, false);
        const auto r1 = __builtin_amdgcn_permlane32_swap((unsigned)W.q[i][1], (unsigned)W.q[i][3], false, false);
        wq[i] = rv2i{(int)r0[0], (int)r1[0]};
        wq[4 + i] = rv2i{(int)r0[1], (int)r1[1]};
      }
      const uint4 hd = make_uint4((uint32_t)W.hd[0], (uint32_t)W.hd[1], (uint32_t)W.hd[2], (uint32_t)W.hd[3]);
      const uint32_t s03 = hd.y & 0x3f3f3f3fu;
      const uint32_t s47 = hd.z & 0x3f3f3f3fu;
      int I[4][NREG];
#pragma unroll
      for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int r = 0; r < NREG; ++r) I[p][r] = 0;
      /* With two wavefronts a SIMD nobody else hides a step's latencies: the eight operands are
       * read from LDS up front, and step j + 1 is issued into a second result register before the
       * sums of step j are taken. */
      rv4i a8[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) a8[j] = *(const rv4i *)(pa + j * 32);
      rv16i D[2];
      auto step = [&](int j) {
        /* weight 2i / 2i+1 of the lane's 16 in the low / high nibble of byte i: the even ones become
         * operand bytes 0-7, the odd ones bytes 8-15 (the order the activations' 16-value groups are
         * stored in) */
        const uint32_t x0 = (uint32_t)wq[j][0], x1 = (uint32_t)wq[j][1];
        const rv4i b = {(int)(x0 & HIPQ_M4), (int)(x1 & HIPQ_M4), (int)((x0 >> 4) & HIPQ_M4),
                        (int)((x1 >> 4) & HIPQ_M4)};
        D[j & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8[j], b, zero16, 0, 0, 0);
      };
      step(0);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (j + 1 < 8) step(j + 1);
        const int scj = (int)(((j < 4 ? s03 : s47) >> (8 * (j & 3))) & 0xff);
#pragma unroll
        for (int r = 0; r < NREG; ++r) I[j >> 1][r] = __mul24(D[j & 1][r], scj) + I[j >> 1][r];
      }
      const uint32_t mlo = (hd.w & 0x0f0f0f0fu) | ((hd.y >> 2) & 0x30303030u);
      const uint32_t mhi = ((hd.w >> 4) & 0x0f0f0f0fu) | ((hd.z >> 2) & 0x30303030u);
      float Sm[4][NREG];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        /* the mins of pair p against the sub-block sums (both halves of the K index carry the same
         * mins: one half meets the sums' low parts, the other the rest) */
        const uint32_t mw = p < 2 ? mlo : mhi;
        rv8h bmin = {0, 0, 0, 0, 0, 0, 0, 0};
        bmin[2 * p] = (_Float16)(float)((mw >> (16 * (p & 1))) & 0xff);
        bmin[2 * p + 1] = (_Float16)(float)((mw >> (16 * (p & 1) + 8)) & 0xff);
        const rv16f S = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < NREG; ++r) Sm[p][r] = S[r];
      }
      uint32_t *rec = lrec + wave * (NREG * 2 * 256) + lane * 4;
#pragma unroll
      for (int r = 0; r < NREG; ++r) {
        *(rv4i *)(rec + (r * 2) * 256) = rv4i{I[0][r], I[1][r], I[2][r], I[3][r]};
        *(rv4i *)(rec + (r * 2 + 1) * 256) =
          rv4i{(int)__float_as_uint(Sm[0][r]), (int)__float_as_uint(Sm[1][r]), (int)__float_as_uint(Sm[2][r]),
               (int)__float_as_uint(Sm[3][r])};
      }
      if (g == 0) {
        ldw[(wave * 2) * 32 + i32] = hipq_h2f((uint16_t)(hd.x & 0xffff));
        ldw[(wave * 2 + 1) * 32 + i32] = hipq_h2f((uint16_t)(hd.x >> 16));
      }
    }
    __syncthreads();
    act_store(AR, (rho + 1) & 1); /* the next round's rows: that buffer was last read a round ago */
    /* the chains of this round's super-blocks, ascending; everything a chain reads is requested
     * before the first step (the records of a wavefront that had no super-block are read as well
     * and not used: a read behind a branch would wait for its own latency) */
    rv4i ivs[SBR], mvs[SBR];
    float dAs[SBR], dws[SBR], dms[SBR];
#pragma unroll
    for (int ws = 0; ws < SBR; ++ws) {
      const uint32_t *rec = lrec + ws * (NREG * 2 * 256) + (cr * 2) * 256 + cl * 4;
      ivs[ws] = *(const rv4i *)rec;
      mvs[ws] = *(const rv4i *)(rec + 256);
      dAs[ws] = ((const float *)(act + ACT_DA))[ws * TC + cm];
      dws[ws] = ldw[(ws * 2) * 32 + cn];
      dms[ws] = ldw[(ws * 2 + 1) * 32 + cn];
    }
#pragma unroll
    for (int ws = 0; ws < SBR; ++ws) {
      const int sbw = rho * SBR + ws;
      if (sbw < nsb) { /* uniform */
        const rv4i iv = ivs[ws], mv = mvs[ws];
        const int I0 = iv[0], I1 = iv[1], I2 = iv[2], I3 = iv[3];
        const float M0 = __int_as_float(mv[0]), M1 = __int_as_float(mv[1]), M2 = __int_as_float(mv[2]),
                    M3 = __int_as_float(mv[3]);
        const float dA = dAs[ws];
        const float sd = dws[ws] * dA, sm = dms[ws] * dA;
        if (pairwise) {
          acc = fmaf((float)I0, sd, acc);
          accm = fmaf(M0, sm, accm);
          acc = fmaf((float)I1, sd, acc);
          accm = fmaf(M1, sm, accm);
          acc = fmaf((float)I2, sd, acc);
          accm = fmaf(M2, sm, accm);
          acc = fmaf((float)I3, sd, acc);
          accm = fmaf(M3, sm, accm);
        } else {
          /* the partial sums of the mins are integers below 2^24: their fp32 sum is exact */
          acc = fmaf((float)(I0 + I1 + I2 + I3), sd, acc);
          accm = fmaf((M0 + M1) + (M2 + M3), sm, accm);
        }
      }
    }
    __syncthreads(); /* the next round overwrites the records */
  };
  /* NB rounds a trip so that each register set has a fixed name; all conditions are uniform */
  for (int rho0 = 0; rho0 < rounds; rho0 += NB) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int rho = rho0 + u;
      if (rho < rounds) {
        act_load(AR, rho + 1); /* before the weights: its wait must not include theirs */
        load(buf[(u + PD) % NB], (rho + PD) * SBR + wave);
        round(buf[u], rho);
      }
    }
  }
  const int col = tile * 32 + cn;
  if (cm < M && col < w.N) C[(int64_t)cm * ldc + col] = acc - accm;
}

} // namespace

namespace hipq {

/* Where it beats the GEMV engine (measured, kernel us old -> new): five to eight rows from 1024
 * columns up (2048 x 1024: 5.5 -> 4.0; 4096 x 4096: 16.4 -> 8.3; 12288 x 4096: 39.0 -> 11.2;
 * 151936 x 4096: 421 -> 75); with fewer rows where the last lines of the rule below say (at first four
 * rows from 4096 columns, 4096 x 4096: 8.7 -> 8.3; 12288 x 4096:
 * 16.4 -> 11.0), three from 8192 (12288 x 4096: 14.2 -> 11; 4096 x 4096: 7.1 against 8.2). A round
 * of a workgroup takes 1.7 us, most of it the issue of its vector instructions (about 290 a
 * wavefront and super-block: nibble expansion, scale multiplies, the chains), so the kernel
 * streams its weights at 2.5-4.6 TB/s. */
bool gemm_rows_q4k_fits(const hipq_weight *w, int64_t M) {
  if (w->dtype != HIPQ_Q4_K || w->expert_tiles || w->K % 256 || 16 * w->K > 0x7fffffff) return false;
  /* More than eight rows: passes of eight side by side in one launch (blockIdx.y). Two passes
   * always (12288 x 4096 with 16 rows: 14.7 us against 17.2 for the prefill GEMM in parts of K; 4096 x
   * 4096: 8.5 against 12.5: a launch of one pass leaves half the chip idle there); up to eight where
   * the launch stays small, measured against that GEMM (us): 4096 x 4096 with 32 / 48 rows 10.1 / 12.5
   * against 12.7 / 13.3, 2048 x 2048 with 64 rows 6.5 against 11.0; but 12288 x 4096 with 24 rows 23.2
   * against 18.3, 4096 x 12288 with 24 rows 24.1 against 18.1. */
  if (M >= 5 && M <= 2 * TC) return w->N >= 1024;
  if (M > 2 * TC && M <= 8 * TC && w->N >= 1024) {
    const int64_t tiles = (w->N + 31) / 32, passes = (M + TC - 1) / TC;
    return tiles * passes * (w->K / 256) <= 8192;
  }
  /* Two to four rows against the engine with its row lengths compiled in (calls in a row on one
   * stream, us, engine / this kernel). Four rows: 4096 x 4096 10.4 / 11.2, 6144 x 4096 11.7 / 11.4,
   * 6144 x 2048 8.6 / 8.5, 12288 x 2048 12.3 / 9.9. Three: 8192 x 4096 11.0 / 11.5, 12288 x 4096 13.5 /
   * 13.4, 32768 x 4096 24.3 / 22.1, 12288 x 2048 11.2 / 9.8, 6144 x 2048 7.9 / 8.4. Two rows stay with
   * the engine (12288 x 4096 10.5 / 13.5, 32768 x 4096 18.0 / 22.0) but for rows of 1024, where the
   * engine's wavefronts hold a quarter of a row each: 16384 x 1024 10.9 / 8.3. */
  const bool long_rows = w->K >= 4096;
  if (M == 4) return w->N >= (long_rows ? 6144 : 4096);
  if (M == 3) return w->N >= (long_rows ? 12288 : 8192);
  return M == 2 && w->K <= 1024 && w->N >= 16384;
}

/* Several weights of one K in one launch (hipq_matmul_multi): what counts is the launch's width, the
 * columns of all of them, and the launches it replaces. */
bool gemm_rows_q4k_fits_multi(int count, const hipq_weight *const *w, int64_t M) {
  if (count < 2 || M < 2 || M > 8 * TC) return false;
  int64_t tiles = 0;
  for (int i = 0; i < count; ++i) {
    if (w[i]->dtype != HIPQ_Q4_K || w[i]->expert_tiles || w[i]->K % 256 || 16 * w[i]->K > 0x7fffffff ||
        w[i]->K != w[0]->K)
      return false;
    tiles += (w[i]->N + 31) / 32;
  }
  if (tiles < 32) return false;
  if (M <= 2 * TC) return true;
  return tiles * ((M + TC - 1) / TC) * (w[0]->K / 256) <= 8192;
}

int launch_gemm_rows_q4k_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, int pair_rows,
                               float *const *C, const int64_t *ldc, hipStream_t s) {
  if (count < 1 || count > 4) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product takes 1 to 4 weights a launch");
  if (M < 1 || M > 8 * TC) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product takes 1..64 rows");
  MultiRowsQ4K mw;
  int tiles = 0;
  for (int i = 0; i < 4; ++i) {
    const int j = i < count ? i : count - 1;
    if (i < count) {
      if (w[i]->dtype != HIPQ_Q4_K || w[i]->expert_tiles || qa->K != w[i]->K || 16 * w[i]->K > 0x7fffffff)
        return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product takes Q4_K weights of the rows' K");
      if (!w[i]->gt_base) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product needs the weight's tile copy");
      tiles += (int)((w[i]->N + 31) / 32);
    }
    mw.w[i] = wview(w[j]);
    mw.w[i].qs = w[j]->gt_qs;
    mw.w[i].hdr = w[j]->gt_hdr;
    mw.C[i] = C[j];
    mw.ldc[i] = ldc[j];
    mw.tile_end[i] = tiles; /* unused entries repeat the total: no workgroup lands in them */
  }
  hipq::launch_kernel("gemm_rows_q4k_kernel", gemm_rows_q4k_kernel, dim3((unsigned)tiles, (unsigned)((M + TC - 1) / TC)), dim3(NT), LDS_BYTES, s, mw,
                     qview(*qa), M, pair_rows);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_gemm_rows_q4k(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
                         hipStream_t s) {
  return launch_gemm_rows_q4k_multi(1, &w, qa, M, pair_rows, &C, &ldc, s);
}

} // namespace hipq
