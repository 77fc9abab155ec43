// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm_rows_q4k.hip
 * @brief  Q4_K x Q8_K for three to eight activation rows on the int8 matrix cores,
 *         with the reference's bits.
 *
 * Replaces, for 3 <= M <= 8, what __ggml_q4_K_8x8_q8_K_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:391-517 in the
 * reference checkout) does with a few rows: the rows below 4 * (M / 4) go through
 * nntr_gemm_q4_K_8x8_q8_K (nntr_ggml_impl.cpp:3261-7078), which adds the four sub-block
 * pairs of a super-block to a row's sum one after the other, the others through
 * nntr_gemv_q4_K_8x8_q8_K (:7080-7494), which adds the super-block's total. The GEMV engine
 * (gemv_device.h) does the same on the vector ALU, where a row of activations costs about
 * 4 us on a 12288 x 4096 matrix (eight rows: 37 us; one row: 8 us, the weight stream); this
 * kernel takes 12.8 us for eight.
 *
 * Here a workgroup owns 32 output columns and all rows. Its four wavefronts take one
 * super-block each per round: one v_mfma_i32_32x32x32_i8 per sub-block (the rows are the
 * row operand: 8 of its 32 rows are used), the 6-bit scales applied to the exact int32 sums
 * pair by pair, the mins through four v_mfma_f32_32x32x16_f16 with all but one pair's mins
 * zeroed. The four partial sums of both kinds go to LDS as they are (integers), and after a
 * barrier every thread runs the fp32 chain of ONE output over the round's super-blocks in
 * ascending order, exactly as the reference orders it, so the chain is as long as on the
 * vector ALU but the integer work is not. Weights come from the 32-row tile copy the prefill
 * GEMM reads (piece i of lane (n, g) = sub-block 4 g + i of row n; the two lanes of a row swap
 * halves with v_permlane32_swap so that each holds its 16 weights of sub-blocks i and 4 + i),
 * the loads of the next two rounds in flight during the current one.
 * Rows of one chunk only (K <= 4096: the quantized rows stay in LDS).
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

struct RowsLds {
  int8_t *q;      /* [TC][K + 16]: rows padded so that the lanes of a 128-bit read fall into different banks */
  uint8_t *amin;  /* [TC][nsb][32 bytes]: sub-block sums as two fp16-exact parts */
  float *dA;      /* [nsb][TC] */
  uint32_t *rec;  /* the round's partial sums */
  float *dw;      /* [SBR][2][32]: d and dmin of the round's super-blocks, per column */
};
__host__ __device__ inline size_t rows_lds_rec_offset(int K) {
  const size_t b = (size_t)TC * (K + 16) + (size_t)TC * (K / 256) * 32 + (size_t)TC * (K / 256) * 4;
  return (b + 255) & ~(size_t)255;
}
__host__ __device__ inline size_t rows_lds_bytes(int K) {
  return rows_lds_rec_offset(K) + (size_t)REC_DWORDS * 4 + (size_t)SBR * 2 * 32 * 4;
}

struct RowsRegs {
  rv4i q[4];
  rv4i hd;
};

__global__ __launch_bounds__(NT, 2) void gemm_rows_q4k_kernel(WView w, QView a, int M, int pair_rows,
                                                              float *__restrict__ C, int64_t ldc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char rows_lds[];
  const int K = w.K, nsb = K >> 8;
  const int tile = blockIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63, i32 = lane & 31, g = lane >> 5;
  RowsLds l;
  l.q = (int8_t *)rows_lds;
  l.amin = rows_lds + (size_t)TC * (K + 16);
  l.dA = (float *)(l.amin + (size_t)TC * nsb * 32);
  l.rec = (uint32_t *)(rows_lds + rows_lds_rec_offset(K));
  l.dw = (float *)(l.rec + REC_DWORDS);

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
  /* The weights of PD + 1 rounds: the loads of the next PD rounds are in flight during a round.
   * Every round issues its loads, past the end those of the last super-block again: with a
   * conditional load the compiler cannot count the loads in flight and waits for all of them. */
  constexpr int PD = 2, NB = PD + 1;
  RowsRegs buf[NB];
  const int rounds = (nsb + SBR - 1) / SBR;
#pragma unroll
  for (int p = 0; p < PD; ++p) load(buf[p], p * SBR + wave);

  /* the M quantized rows, while the first weights are on their way (rows M .. TC - 1 of the
   * matrix operand keep what the LDS held: a row of the product depends on its own
   * activations only, and those rows are not stored) */
  {
    const int cpr = K >> 4, np = M * cpr;
    /* four loads before their stores, so that their latencies overlap */
    for (int c0 = threadIdx.x; c0 < np; c0 += 4 * NT) {
      rv4i v[4];
      int dst[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = min(c0 + u * NT, np - 1);
        const int r = c / cpr, o = c - r * cpr;
        v[u] = *(const rv4i *)(a.q + (size_t)r * K + o * 16);
        dst[u] = r * (K + 16) + o * 16;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c0 + u * NT < np) *(rv4i *)(l.q + dst[u]) = v[u];
    }
    for (int c = threadIdx.x; c < M * nsb * 2; c += NT)
      *(rv4i *)(l.amin + c * 16) = *(const rv4i *)((const uint8_t *)a.bsum + (size_t)c * 16);
    for (int c = threadIdx.x; c < M * nsb; c += NT) {
      const int r = c / nsb, b = c - r * nsb;
      l.dA[b * TC + r] = a.d[c];
    }
  }
  __syncthreads();

  /* the output this thread chains: row cm, column cn; its sums sit in register cr of lane cl */
  const int cn = threadIdx.x & 31, cm = threadIdx.x >> 5;
  const int cr = cm & 3, cl = (cm >> 2) * 32 + cn;
  const bool pairwise = cm < pair_rows;
  float acc = 0.f, accm = 0.f;

  auto round = [&](const RowsRegs &W, int rho) {
    const int sb = rho * SBR + wave;
    if (sb < nsb) { /* uniform per wavefront */
      const rv16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const rv16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const int row = i32 & (TC - 1);
      const int8_t *pa = l.q + row * (K + 16) + sb * 256 + g * 16;
      const rv8h amin = *(const rv8h *)(l.amin + (row * nsb + sb) * 32 + g * 16);
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
      uint32_t *rec = l.rec + wave * (NREG * 2 * 256) + lane * 4;
#pragma unroll
      for (int r = 0; r < NREG; ++r) {
        *(rv4i *)(rec + (r * 2) * 256) = rv4i{I[0][r], I[1][r], I[2][r], I[3][r]};
        *(rv4i *)(rec + (r * 2 + 1) * 256) =
          rv4i{(int)__float_as_uint(Sm[0][r]), (int)__float_as_uint(Sm[1][r]), (int)__float_as_uint(Sm[2][r]),
               (int)__float_as_uint(Sm[3][r])};
      }
      if (g == 0) {
        l.dw[(wave * 2) * 32 + i32] = hipq_h2f((uint16_t)(hd.x & 0xffff));
        l.dw[(wave * 2 + 1) * 32 + i32] = hipq_h2f((uint16_t)(hd.x >> 16));
      }
    }
    __syncthreads();
    /* the chains of this round's super-blocks, ascending; everything a chain reads is requested
     * before the first step (the records of a wavefront that had no super-block are read as well
     * and not used: a read behind a branch would wait for its own latency) */
    rv4i ivs[SBR], mvs[SBR];
    float dAs[SBR], dws[SBR], dms[SBR];
#pragma unroll
    for (int ws = 0; ws < SBR; ++ws) {
      const uint32_t *rec = l.rec + ws * (NREG * 2 * 256) + (cr * 2) * 256 + cl * 4;
      ivs[ws] = *(const rv4i *)rec;
      mvs[ws] = *(const rv4i *)(rec + 256);
      dAs[ws] = l.dA[min(rho * SBR + ws, nsb - 1) * TC + cm];
      dws[ws] = l.dw[(ws * 2) * 32 + cn];
      dms[ws] = l.dw[(ws * 2 + 1) * 32 + cn];
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
 * columns up (2048 x 1024: 5.5 -> 4.8; 4096 x 4096: 16.4 -> 9.2; 12288 x 4096: 39.0 -> 12.8;
 * 151936 x 4096: 421 -> 94), three and four rows on large matrices only (12288 x 4096: 14.2 and
 * 16.4 -> 12.2; 4096 x 4096: 7.1 and 8.7 against 9). A round of a workgroup takes 1.7 us, most of
 * it the issue of its vector instructions (about 290 a wavefront and super-block: nibble
 * expansion, scale multiplies, the chains), so the kernel runs at 2-3.6 TB/s of weights. */
bool gemm_rows_q4k_fits(const hipq_weight *w, int64_t M) {
  if (w->dtype != HIPQ_Q4_K || w->expert_tiles || w->K > HIPQ_KCHUNK || w->K % 256) return false;
  if (M >= 5 && M <= TC) return w->N >= 1024;
  return (M == 3 || M == 4) && w->N >= 8192;
}

int launch_gemm_rows_q4k(const hipq_weight *w, const QAct *qa, int M, int pair_rows, float *C, int64_t ldc,
                         hipStream_t s) {
  if (!gemm_rows_q4k_fits(w, M) || qa->K != w->K)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product takes 3..8 rows of one chunk");
  if (!w->gt_base) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the few-rows Q4_K product needs the weight's tile copy");
  const size_t lds = rows_lds_bytes((int)w->K);
  if (lds > 64 * 1024)
    HIPQ_HIP(hipFuncSetAttribute((const void *)gemm_rows_q4k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                 (int)lds));
  WView v = wview(w);
  v.qs = w->gt_qs;
  v.hdr = w->gt_hdr;
  const unsigned grid = (unsigned)((w->N + 31) / 32);
  hipLaunchKernelGGL(gemm_rows_q4k_kernel, dim3(grid), dim3(NT), lds, s, v, qview(*qa), M, pair_rows, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
