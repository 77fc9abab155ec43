// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm_q4k.hip
 * @brief  Prefill GEMM for Q4_K x Q8_K on the gfx950 int8 matrix cores.
 *
 * Replaces the M > 1 branch of __ggml_q4_K_8x8_q8_K_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:432-486 in
 * the reference checkout) and nntr_gemm_q4_K_8x8_q8_K behind it
 * (nntr_ggml_impl/nntr_ggml_impl.cpp:3261-7078). Per output and super-block the
 * reference needs  I = sum_j sc_j * (q4 . q8)_j  with eight 6-bit sub-block
 * scales sc_j. Scaling each 32-deep MFMA result on the vector ALU costs one
 * multiply-add per result and caps an int8 kernel far below the matrix peak
 * (the ALU retires 16 lane-ops per cycle and SIMD, the matrix core 1024 MACs).
 * Here the scale goes into the weights instead. A product sc*q4 <= 945 does not
 * fit int8, but with sc = 8*hi3 + lo3 both digit planes q4*lo3 and q4*hi3
 * (<= 105) do, and
 *       I = sum_k (q4*lo3)[k] * q8[k]  +  8 * sum_k (q4*hi3)[k] * q8[k]
 * accumulates over the whole 256-deep super-block inside the matrix core: two
 * chains of v_mfma_i32_32x32x32_i8, exact int32, no per-sub-block ALU work.
 * The min term  Im = sum_j m_j * bsum_j  (K = 8 per super-block) is one
 * v_mfma_f32_32x32x16_f16 with bsum split into two fp16-exact parts; its fp32
 * result is exact (< 2^24). Per super-block and output the ALU does
 *       acc += dA * (d * float(Dlo + 8*Dhi) - dmin * Im).
 *
 * Tiling. A workgroup (4 wavefronts side by side) owns a 64 x 128 or 128 x 128 tile
 * of C, each wavefront all its rows x 32 columns (2 or 4 MFMA row tiles x 2 digit
 * chains). K is walked in stages of 128. Three workgroups of the 64-row kind share
 * a CU (29 KB of LDS, at most 168 registers), so one's matrix phase overlaps the
 * others' vector work and the 768 tiles of the 512 x 12288 reference shape are all
 * resident at once; of the 128-row kind two fit (57 KB, 256 registers), which do a
 * fifth more work per unit of time because the weight expansion is shared by twice
 * the rows. The launcher picks by the number of rounds the grid takes.
 *  - Weights never pass through LDS: a wavefront owns its 32 columns for the whole
 *    of K, lane (n, g) reads the 64 bytes of sub-blocks 4g .. 4g+3 of column n one
 *    stage ahead (ordinary loads: two lanes share a 128-byte line) and expands 16
 *    weights per 32-deep step into the two digit planes in registers: the even ones
 *    (low nibbles) become operand bytes 0-7, the odd ones bytes 8-15. So there is no
 *    workgroup-wide expansion phase and no barrier on the weights' account.
 *  - Activations come from the quantizer already in that operand order, 16 KB per
 *    128 rows and 128-deep stage (hipq_internal.h, QActTiled), and go from HBM/L2
 *    straight into a three-slot LDS ring with buffer_load_dwordx4 ... lds, two
 *    stages ahead: no registers, no ALU work, and the ds_read_b128 of a wavefront
 *    covers 1 KB of consecutive LDS. (The buffer form matters: after a global
 *    direct-to-LDS load the compiler waits for every load in flight at the next
 *    use of any loaded register.) One barrier per stage hands a ring slot over.
 *  - The per-row data of a super-block (bsum parts, d) is copied the same way.
 * Workgroup ids are mapped so that the M-tiles sharing a weight tile run on the
 * same XCD (same L2).
 */
#include "gemv_device.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int BN = 128;
constexpr int NT = 256;           /* 4 wavefronts side by side, 32 columns each */
constexpr int QSTAGE = 128 * 128; /* bytes of one stage as the quantizer writes it (128 rows) */

/* LDS of a workgroup whose wavefronts hold TM row tiles of 32 (tile height 32 * TM) */
template <int TM> struct Smem {
  static constexpr int BM = 32 * TM;
  static constexpr int ASTAGE = BM * 128; /* bytes of one 128-deep activation stage of the tile */
  int8_t a[3][ASTAGE];       /* ring of stages, each [row/32][step 4][lane 64][16] */
  _Float16 amin[2][BM * 16]; /* per super-block: per row 8 low parts, 8 high parts of bsum32_j */
  float dA[2][BM];
};
static_assert(sizeof(Smem<2>) * 3 <= 160 * 1024 && sizeof(Smem<4>) * 2 <= 160 * 1024,
              "three workgroups of 64 rows or two of 128 rows per CU must fit the 160 KB LDS");

__device__ __forceinline__ uint32_t pk_scale(uint32_t x, uint32_t digit2) {
  const v2us r = __builtin_bit_cast(v2us, x) * __builtin_bit_cast(v2us, digit2);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ void dma16(rsrc_t r, uint32_t voff, uint32_t soff, void *lds_wave) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_wave, 16,
                                           (int)voff, (int)soff, 0, 0);
}
__device__ __forceinline__ void dma4(rsrc_t r, uint32_t voff, uint32_t soff, void *lds_wave) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)lds_wave, 4,
                                           (int)voff, (int)soff, 0, 0);
}
template <int VM> __device__ __forceinline__ void sync_lds() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

struct Src {
  rsrc_t qt, amin, dAt;
  const uint4 *wq, *whd; /* plane layout: this lane's 64 bytes of nibbles / header of super-block 0 */
  rsrc_t rq, rh;         /* tile copy: the wavefront's tile, nibbles / headers; the descriptors sit in scalar
                            registers and a load names a lane offset and a scalar offset (no per-lane
                            64-bit pointers to keep or to add to) */
  int wave, lane;
};
typedef unsigned int u4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16(rsrc_t r, uint32_t voff, uint32_t soff) {
  const u4v v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
  return make_uint4(v[0], v[1], v[2], v[3]);
}
struct WHalf { /* this lane's two sub-blocks of one 128-deep stage */
  uint4 q[2];
};
/* TILES: the weights come from the tile copy (hipq_internal.h, gt_qs): piece i of lane
 * (n, g) is sub-block 4g + i, 64 lanes x 16 bytes consecutive per piece, so a load
 * instruction covers 1 KB of memory instead of 32 separate lines. */
template <bool TILES> __device__ __forceinline__ void load_wh(WHalf &W, const Src &sr, int sb, int h) {
  if (TILES) {
    W.q[0] = ld16(sr.rq, sr.lane * 16, (uint32_t)(sb * 4 + 2 * h) * 1024);
    W.q[1] = ld16(sr.rq, sr.lane * 16, (uint32_t)(sb * 4 + 2 * h + 1) * 1024);
  } else {
    W.q[0] = hipq_ld_global(sr.wq + sb * 8 + 2 * h);
    W.q[1] = hipq_ld_global(sr.wq + sb * 8 + 2 * h + 1);
  }
}
/* stage (128 deep) -> ring slot: each wavefront copies a quarter of the tile's stage, TM KB */
template <int TM>
__device__ __forceinline__ void dma_a(const Src &sr, Smem<TM> &sm, int stage, int slot) {
  const uint32_t so = (uint32_t)stage * QSTAGE + sr.wave * (TM * 1024);
  int8_t *l = sm.a[slot] + sr.wave * (TM * 1024);
#pragma unroll
  for (int i = 0; i < TM; ++i) dma16(sr.qt, sr.lane * 16, so + i * 1024, l + i * 1024);
}
/* per-row data of a super-block: 32 bytes of bsum parts and one scale per row */
template <int TM>
__device__ __forceinline__ void dma_rows(const Src &sr, Smem<TM> &sm, int sb, int buf) {
  if (sr.wave < TM) /* uniform per wavefront */
    dma16(sr.amin, sr.lane * 16, (uint32_t)sb * (128 * 32) + sr.wave * 1024, (char *)sm.amin[buf] + sr.wave * 1024);
  if (TM == 2 ? sr.wave == 2 : sr.wave < 2)
    dma4(sr.dAt, sr.lane * 4, (uint32_t)sb * (128 * 4) + (TM == 2 ? 0 : sr.wave * 256),
         sm.dA[buf] + (TM == 2 ? 0 : sr.wave * 64));
}
/* Loads a wavefront issues at least per stage (some wavefronts copy no per-row
 * data): what may stay in flight at the stage's barrier. First / second half. */
template <int TM> struct InFlight {
  static constexpr int FIRST = TM + (TM == 2 ? 0 : 1) + 2; /* copies of the ring, row data, two nibble loads */
  static constexpr int SECOND = TM + 3;                    /* copies of the ring, two nibble loads, the header */
};

/* four 32-deep steps of one 128-deep stage: H = which half of the super-block */
template <int H, int TM>
__device__ __forceinline__ void stage_mma(const Smem<TM> &sm, int slot, const WHalf &W, uint32_t slo, uint32_t shi,
                                          int lane, v16i (&Dlo)[TM], v16i (&Dhi)[TM]) {
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int8_t *pa = sm.a[0] + slot * Smem<TM>::ASTAGE + lane * 16;
  v4i a[2][TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) a[0][tm] = *(const v4i *)(pa + (tm * 4) * 1024);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const int s = H * 4 + ks, j = s >> 1, half = s & 1; /* this lane's sub-block 4g + j, 16 weights */
    if (ks + 1 < 4) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) a[(ks + 1) & 1][tm] = *(const v4i *)(pa + (tm * 4 + ks + 1) * 1024);
    }
    const uint32_t dl = __builtin_amdgcn_perm(slo, slo, 0x0c000c00u | (uint32_t)j | ((uint32_t)j << 16));
    const uint32_t dh = __builtin_amdgcn_perm(shi, shi, 0x0c000c00u | (uint32_t)j | ((uint32_t)j << 16));
    const uint32_t x0 = half ? W.q[j & 1].z : W.q[j & 1].x, x1 = half ? W.q[j & 1].w : W.q[j & 1].y;
    const uint32_t e0 = x0 & HIPQ_M4, e1 = x1 & HIPQ_M4, o0 = (x0 >> 4) & HIPQ_M4, o1 = (x1 >> 4) & HIPQ_M4;
    const v4i bl = {(int)pk_scale(e0, dl), (int)pk_scale(e1, dl), (int)pk_scale(o0, dl), (int)pk_scale(o1, dl)};
    const v4i bh = {(int)pk_scale(e0, dh), (int)pk_scale(e1, dh), (int)pk_scale(o0, dh), (int)pk_scale(o1, dh)};
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      Dlo[tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks & 1][tm], bl, (H == 0 && ks == 0) ? zero16 : Dlo[tm], 0, 0, 0);
      Dhi[tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks & 1][tm], bh, (H == 0 && ks == 0) ? zero16 : Dhi[tm], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <int TM>
__device__ __forceinline__ void epilogue(const Smem<TM> &sm, int buf, const uint4 &hd, int lane, const v16i (&Dlo)[TM],
                                         const v16i (&Dhi)[TM], float (&acc)[TM][16]) {
  const v16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int i32 = lane & 31, g = lane >> 5;
  const float dcol = hipq_h2f((uint16_t)(hd.x & 0xffff));
  const float ndmin = -hipq_h2f((uint16_t)(hd.x >> 16));
  const uint32_t mlo = (hd.w & 0x0f0f0f0fu) | ((hd.y >> 2) & 0x30303030u);
  const uint32_t mhi = ((hd.w >> 4) & 0x0f0f0f0fu) | ((hd.z >> 2) & 0x30303030u);
  v8h bmin;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    bmin[j] = (_Float16)(float)((mlo >> (8 * j)) & 0xff);
    bmin[4 + j] = (_Float16)(float)((mhi >> (8 * j)) & 0xff);
  }
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int rbase = tm * 32;
    const v8h amin = __builtin_bit_cast(v8h, *(const v4i *)((const int8_t *)sm.amin[buf] + ((rbase + i32) * 16 + g * 8) * 2));
    const v16f Sm = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const v4i dv = *(const v4i *)((const int8_t *)sm.dA[buf] + (rbase + 8 * q4 + 4 * g) * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * q4 + e;
        const int I = (Dhi[tm][r] << 3) + Dlo[tm][r];
        float tt = dcol * (float)I;
        tt = fmaf(ndmin, Sm[r], tt);
        acc[tm][r] = fmaf(__int_as_float(dv[e]), tt, acc[tm][r]);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(acc[tm][r]));
    __builtin_amdgcn_sched_barrier(0);
  }
}

/* the tile (mt, nt) of one weight's product */
/* KSPLIT: the tile's sum over super-blocks sb0 .. sb0 + nsbl - 1 only (a partial product; the
 * callers add the parts). Everything the loop reads is addressed relative to its first
 * super-block, so the part's first one becomes that by moving the bases. */
template <int TM, bool TILES, bool KSPLIT = false>
__device__ __forceinline__ void gemm_q4k_tile(const WView &w, const int8_t *__restrict__ qt,
                                              const uint16_t *__restrict__ amin, const float *__restrict__ dAt, int M,
                                              int mt, int nt, float *__restrict__ C, int64_t ldc, int sb0 = 0,
                                              int nsb_part = 0) {
  static_assert(!KSPLIT || TILES, "partial products read the tile copy");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem<TM> &sm = *reinterpret_cast<Smem<TM> *>(smem_raw);
  constexpr int BM = 32 * TM;
  const int m0 = mt * BM, n0 = nt * BN;
  const int nsb_all = w.K >> 8;
  const int first = KSPLIT ? sb0 : 0;
  const int nsb = KSPLIT ? nsb_part : nsb_all; /* the super-blocks this call walks */
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int i32 = lane & 31, g = lane >> 5;

  Src sr;
  /* the quantizer tiles by 128 rows: a 64-row tile is half mt & 1 of quantizer tile mt / 2 */
  const int qt128 = TM == 2 ? mt >> 1 : mt, hrow = TM == 2 ? mt & 1 : 0;
  sr.qt = make_rsrc(qt + ((size_t)qt128 * (2 * nsb_all) + 2 * first) * QSTAGE + hrow * 8192, (uint32_t)(2 * nsb) * QSTAGE);
  sr.amin = make_rsrc(amin + (((size_t)qt128 * nsb_all + first) * 128 + hrow * 64) * 16, (uint32_t)nsb * 128 * 32);
  sr.dAt = make_rsrc(dAt + ((size_t)qt128 * nsb_all + first) * 128 + hrow * 64, (uint32_t)nsb * 128 * 4);
  const int n = min(n0 + wave * 32 + i32, (int)w.N - 1);
  constexpr int HSTRIDE = TILES ? 32 : 1; /* uint4 between a column's consecutive super-block headers */
  if (TILES) {
    /* the copy pads N to 32 rows: a wavefront whose columns start below N has its tile */
    const size_t wt = (size_t)(min(n0 + wave * 32, (int)w.N - 1) >> 5);
    sr.rq = make_rsrc(w.qs + (wt * nsb_all + first) * 4096, (uint32_t)nsb * 4096);
    sr.rh = make_rsrc(w.hdr + (wt * nsb_all + first) * 512, (uint32_t)nsb * 512);
    sr.wq = nullptr;
    sr.whd = nullptr;
  } else {
    sr.wq = (const uint4 *)(w.qs + (size_t)n * (w.K >> 1) + g * 64);
    sr.whd = (const uint4 *)w.hdr + (size_t)n * nsb_all;
  }
  sr.wave = wave;
  sr.lane = lane;

  v16i Dlo[TM], Dhi[TM];
  float acc[TM][16];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  WHalf Wa, Wb; /* first / second half of a super-block */
  uint4 hd0, hd1;
  load_wh<TILES>(Wa, sr, 0, 0);
  hd0 = TILES ? ld16(sr.rh, i32 * 16, 0) : hipq_ld_global(sr.whd);
  dma_rows(sr, sm, 0, 0);
  dma_a(sr, sm, 0, 0);
  dma_a(sr, sm, 1, 1);
  sync_lds<0>();
  int slot = 0; /* ring slot of the current stage */
  const int nstage = 2 * nsb;
  /* One super-block = two 128-deep stages. Each stage first issues what later
   * stages need (the copy of the stage after next into the ring slot read last,
   * the other half's nibbles, once per super-block the next one's row data and
   * header), then runs its four matrix steps; the barrier at its end waits for the
   * loads issued BEFORE this stage (they retire in order) and leaves this stage's in
   * flight. hd / hdn and Wa / Wb alternate between consecutive super-blocks. */
  auto super_block = [&](int sb, const uint4 &hd, uint4 &hdn, int eb) {
    /* 6-bit scales of sub-blocks 4g .. 4g+3, one per byte, as two 3-bit digits */
    const uint32_t sc = (g ? hd.z : hd.y) & 0x3f3f3f3fu;
    const uint32_t slo = sc & 0x07070707u, shi = (sc >> 3) & 0x07070707u;
    const int sbn = min(sb + 1, nsb - 1);
    {
      const int s2 = slot >= 1 ? slot - 1 : 2; /* the slot read last stage */
      dma_a(sr, sm, min(2 * sb + 2, nstage - 1), s2);
      dma_rows(sr, sm, sbn, eb ^ 1);
      load_wh<TILES>(Wb, sr, sb, 1);
      stage_mma<0>(sm, slot, Wa, slo, shi, lane, Dlo, Dhi);
      slot = slot == 2 ? 0 : slot + 1;
      sync_lds<InFlight<TM>::FIRST>();
    }
    {
      const int s2 = slot >= 1 ? slot - 1 : 2;
      dma_a(sr, sm, min(2 * sb + 3, nstage - 1), s2);
      load_wh<TILES>(Wa, sr, sbn, 0);
      hdn = TILES ? ld16(sr.rh, i32 * 16, (uint32_t)sbn * 512) : hipq_ld_global(sr.whd + sbn * HSTRIDE);
      stage_mma<1>(sm, slot, Wb, slo, shi, lane, Dlo, Dhi);
      slot = slot == 2 ? 0 : slot + 1;
    }
    epilogue(sm, eb, hd, lane, Dlo, Dhi, acc);
    sync_lds<InFlight<TM>::SECOND>();
  };
  int sb = 0;
  for (; sb + 1 < nsb; sb += 2) {
    super_block(sb, hd0, hd1, 0);
    super_block(sb + 1, hd1, hd0, 1);
  }
  if (sb < nsb) super_block(sb, hd0, hd1, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  const int ncol = n0 + wave * 32 + i32;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + tm * 32 + acc_row(r, lane);
      if (m < M && ncol < w.N) C[(int64_t)m * ldc + ncol] = acc[tm][r];
    }
}

template <int TM, bool TILES>
__global__ __launch_bounds__(NT, TM == 2 ? 3 : 2) void gemm_q4k_kernel(WView w, const int8_t *__restrict__ qt,
                                                         const uint16_t *__restrict__ amin,
                                                         const float *__restrict__ dAt, int M, int mtiles,
                                                         int ntiles, float *__restrict__ C, int64_t ldc) {
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles, nt = (qd / mtiles) * 8 + xcd;
  if (nt >= ntiles) return; /* uniform per workgroup */
  gemm_q4k_tile<TM, TILES>(w, qt, amin, dAt, M, mt, nt, C, ldc);
}

/* Few tiles (up to 64 rows against a matrix of a few thousand columns make under a hundred
 * workgroups, each walking all of K: 31 us at 12288 x 4096 whatever the row count): blockIdx.y
 * takes a part of K and writes its partial product to part[y]; split_sum_kernel adds the parts
 * in ascending order. */
__global__ __launch_bounds__(NT, 3) void gemm_q4k_split_kernel(WView w, const int8_t *__restrict__ qt,
                                                               const uint16_t *__restrict__ amin,
                                                               const float *__restrict__ dAt, int M, int mtiles,
                                                               int ntiles, int sb_per_part, float *__restrict__ part,
                                                               int64_t part_stride) {
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles, nt = (qd / mtiles) * 8 + xcd;
  if (nt >= ntiles) return; /* uniform per workgroup */
  const int sb0 = blockIdx.y * sb_per_part;
  const int n = min(sb_per_part, (w.K >> 8) - sb0);
  gemm_q4k_tile<2, true, true>(w, qt, amin, dAt, M, mt, nt, part + (int64_t)blockIdx.y * part_stride, w.N, sb0, n);
}

__global__ __launch_bounds__(256) void split_sum_kernel(const float *__restrict__ part, int parts, int64_t part_stride,
                                                        int M, int N, float *__restrict__ C, int64_t ldc) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4; /* N % 4 == 0 */
  if (i >= (int64_t)M * N) return;
  const int m = (int)(i / N), n = (int)(i - (int64_t)m * N);
  float4 v = *(const float4 *)(part + i);
  for (int p = 1; p < parts; ++p) {
    const float4 u = *(const float4 *)(part + p * part_stride + i);
    v.x += u.x, v.y += u.y, v.z += u.z, v.w += u.w;
  }
  *(float4 *)(C + (int64_t)m * ldc + n) = v;
}

/* Up to four weights of one K (each with its tile copy) against the same activations as ONE
 * launch: the column tiles of the weights follow each other in the grid (Q, K, V of a layer with
 * grouped-query attention: two of the three grids would be an eighth of the chip each). */
struct MultiQ4K {
  WView w[4];
  float *C[4];
  int64_t ldc[4];
  int tile_end[4]; /* running sum of the weights' column tiles */
};
template <int TM>
__global__ __launch_bounds__(NT, TM == 2 ? 3 : 2) void gemm_q4k_multi_kernel(MultiQ4K mw, const int8_t *__restrict__ qt,
                                                               const uint16_t *__restrict__ amin,
                                                               const float *__restrict__ dAt, int M, int mtiles) {
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles;
  int nt = (qd / mtiles) * 8 + xcd;
  if (nt >= mw.tile_end[3]) return; /* uniform per workgroup */
  int wi = 0;
  if (nt >= mw.tile_end[0]) wi = 1;
  if (nt >= mw.tile_end[1]) wi = 2;
  if (nt >= mw.tile_end[2]) wi = 3;
  if (wi) nt -= mw.tile_end[wi - 1];
  const WView w = wi == 0 ? mw.w[0] : wi == 1 ? mw.w[1] : wi == 2 ? mw.w[2] : mw.w[3];
  float *C = wi == 0 ? mw.C[0] : wi == 1 ? mw.C[1] : wi == 2 ? mw.C[2] : mw.C[3];
  const int64_t ldc = wi == 0 ? mw.ldc[0] : wi == 1 ? mw.ldc[1] : wi == 2 ? mw.ldc[2] : mw.ldc[3];
  gemm_q4k_tile<TM, true>(w, qt, amin, dAt, M, mt, nt, C, ldc);
}

} // namespace

namespace hipq {

template <int TM>
int launch_tiles(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  const int mtiles = (M + 32 * TM - 1) / (32 * TM);
  const int ntiles = (int)((w->N + BN - 1) / BN);
  const int ngroups = (ntiles + 7) / 8;
  const unsigned grid = (unsigned)(mtiles * ngroups * 8);
  WView v = wview(w);
  if (w->gt_base) { /* the tile copy, where the weight has one */
    v.qs = w->gt_qs;
    v.hdr = w->gt_hdr;
    hipq::launch_kernel(TM == 2 ? "gemm_q4k_kernel<2, true>" : "gemm_q4k_kernel<4, true>", gemm_q4k_kernel<TM, true>, dim3(grid), dim3(NT), sizeof(Smem<TM>), s, v, (const int8_t *)qa->qt,
                  (const uint16_t *)qa->amin, (const float *)qa->dAt, M, mtiles, ntiles, C, ldc);
  } else
    hipq::launch_kernel(TM == 2 ? "gemm_q4k_kernel<2, false>" : "gemm_q4k_kernel<4, false>", gemm_q4k_kernel<TM, false>, dim3(grid), dim3(NT), sizeof(Smem<TM>), s, v, (const int8_t *)qa->qt,
                  (const uint16_t *)qa->amin, (const float *)qa->dAt, M, mtiles, ntiles, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* count weights (2 to 4) of one K, every one with its tile copy, as one launch */
int launch_gemm_q4k_multi(int count, const hipq_weight *const *w, const QActTiled *qa, int M, float *const *C,
                          const int64_t *ldc, hipStream_t s) {
  if (count < 1 || count > 4) return fail(HIPQ_ERR_INVALID_ARGUMENT, "1 to 4 weights per launch, got %d", count);
  if ((M + 127) / 128 != qa->mtiles) return fail(HIPQ_ERR_INVALID_ARGUMENT, "tiled activations do not match the matmul shape");
  MultiQ4K mw;
  int tiles = 0;
  for (int i = 0; i < 4; ++i) {
    const hipq_weight *wi = w[i < count ? i : count - 1];
    if (i < count) {
      if (wi->dtype != HIPQ_Q4_K || !wi->gt_base || wi->K != qa->K)
        return fail(HIPQ_ERR_INVALID_ARGUMENT, "the weights of one launch are Q4_K with a tile copy and share K");
      tiles += (int)((wi->N + BN - 1) / BN);
    }
    mw.w[i] = wview(wi);
    mw.w[i].qs = wi->gt_qs;
    mw.w[i].hdr = wi->gt_hdr;
    mw.C[i] = C[i < count ? i : count - 1];
    mw.ldc[i] = ldc[i < count ? i : count - 1];
    mw.tile_end[i] = tiles;
  }
  const int64_t rounds64 = (((int64_t)(M + 63) / 64) * tiles + 767) / 768;
  const int64_t rounds128 = (((int64_t)(M + 127) / 128) * tiles + 511) / 512;
  const int ngroups = (tiles + 7) / 8;
  if (rounds128 * 6 < rounds64 * 5) {
    const int mtiles = (M + 127) / 128;
    hipq::launch_kernel("gemm_q4k_multi_kernel<4>", gemm_q4k_multi_kernel<4>, dim3((unsigned)(mtiles * ngroups * 8)), dim3(NT), sizeof(Smem<4>), s, mw,
                       (const int8_t *)qa->qt, (const uint16_t *)qa->amin, (const float *)qa->dAt, M, mtiles);
  } else {
    const int mtiles = (M + 63) / 64;
    hipq::launch_kernel("gemm_q4k_multi_kernel<2>", gemm_q4k_multi_kernel<2>, dim3((unsigned)(mtiles * ngroups * 8)), dim3(NT), sizeof(Smem<2>), s, mw,
                       (const int8_t *)qa->qt, (const uint16_t *)qa->amin, (const float *)qa->dAt, M, mtiles);
  }
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* Parts of K for a product whose 64-row tiles would leave most of the chip idle (0: none), and
 * the bytes of partial products they need. */
int gemm_q4k_split_parts(const hipq_weight *w, int64_t M) {
  if (w->dtype != HIPQ_Q4_K || !w->gt_base || (w->N & 3)) return 0;
  const int64_t tiles = ((M + 63) / 64) * ((w->N + BN - 1) / BN), nsb = w->K / 256;
  /* measured at 12288 x 4096 (us, whole K a workgroup -> parts): 17..64 rows 31 -> 17-20, 128 rows
   * 33 -> 28; with more than 192 tiles the parts cost what they gain (256 rows 39.4 -> 40.8) */
  if (tiles > 192 || nsb < 8) return 0;
  int parts = (int)(768 / tiles); /* three workgroups a CU */
  if (parts > 8) parts = 8;
  if (parts > nsb / 4) parts = (int)(nsb / 4);
  return parts >= 2 ? parts : 0;
}
size_t gemm_q4k_split_bytes(const hipq_weight *w, int64_t M) {
  return (size_t)gemm_q4k_split_parts(w, M) * (size_t)M * (size_t)w->N * 4;
}

int launch_gemm_q4k(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc, hipStream_t s,
                    void *partials) {
  if ((M + 127) / 128 != qa->mtiles || qa->K != w->K)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "tiled activations do not match the matmul shape");
  const int parts = partials ? gemm_q4k_split_parts(w, M) : 0;
  if (parts && !(ldc & 3) && !((uintptr_t)C & 15)) {
    const int nsb = (int)(w->K / 256), per = (nsb + parts - 1) / parts;
    const int mtiles = (M + 63) / 64, ntiles = (int)((w->N + BN - 1) / BN), ngroups = (ntiles + 7) / 8;
    const int64_t stride = (int64_t)M * w->N;
    WView v = wview(w);
    v.qs = w->gt_qs;
    v.hdr = w->gt_hdr;
    hipq::launch_kernel("gemm_q4k_split_kernel", gemm_q4k_split_kernel, dim3((unsigned)(mtiles * ngroups * 8), (unsigned)((nsb + per - 1) / per)),
                  dim3(NT), sizeof(Smem<2>), s, v, (const int8_t *)qa->qt, (const uint16_t *)qa->amin,
                  (const float *)qa->dAt, M, mtiles, ntiles, per, (float *)partials, stride);
    HIPQ_HIP(hipGetLastError());
    const int64_t quads = stride / 4;
    hipq::launch_kernel("split_sum_kernel", split_sum_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s,
                       (const float *)partials, (nsb + per - 1) / per, stride, M, (int)w->N, C, ldc);
    HIPQ_HIP(hipGetLastError());
    return HIPQ_OK;
  }
  /* 128-row tiles do a fifth more work per CU and time (the weight expansion is
   * shared by twice the rows) but only two workgroups fit a CU: 512 tiles per round
   * against 768 of the 64-row kind. Pick by the number of rounds. */
  const int64_t nt = (w->N + BN - 1) / BN;
  const int64_t rounds64 = (((int64_t)(M + 63) / 64) * nt + 767) / 768;
  const int64_t rounds128 = (((int64_t)(M + 127) / 128) * nt + 511) / 512;
  if (rounds128 * 6 < rounds64 * 5) return launch_tiles<4>(w, qa, M, C, ldc, s);
  return launch_tiles<2>(w, qa, M, C, ldc, s);
}

} // namespace hipq
