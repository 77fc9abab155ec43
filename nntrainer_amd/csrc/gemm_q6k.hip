// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm_q6k.hip
 * @brief  Prefill GEMM for Q6_K x Q8_K on the gfx950 int8 matrix cores.
 *
 * Replaces the M > 1 use of __ggml_gemm_q6_K
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_mixed.cpp:776-821 in the
 * reference checkout: M x N calls of nntr_vec_dot_q6_K_q8_K,
 * nntr_ggml_impl/nntr_ggml_impl.cpp:8280-9514). Per output and super-block the reference
 * needs  I = sum_j scale_j * sum_16 (q6 - 32) * q8  with sixteen int8 sub-block scales.
 * As in the Q4_K kernel the scale goes into the weight operand, so that the matrix core
 * accumulates over the whole 256-deep super-block. The product v = (q6 - 32) * scale
 * (|v| <= 4064) does not fit int8 and neither factor splits into digits whose products do
 * (one of them has eight bits), so the PRODUCT is split into a signed low byte and a signed
 * high byte:  4 v = 256 * h + l  (the factor 4 puts the split on a byte boundary of the
 * 16-bit lanes the product is formed in, see scale_split), and
 *       4 I = sum_k l[k] * q8[k]  +  256 * sum_k h[k] * q8[k]
 * is two chains of v_mfma_i32_32x32x32_i8, exact int32 (|4 I| < 2^30). There is no min term
 * (the format is symmetric). Per super-block and output the ALU does
 *       acc += dA * ((d / 4) * float(Dl + 256 Dh)).
 *
 * The expansion works on 16-bit lanes, two weights per instruction: per four weights two
 * byte selections into lanes, two multiply-adds, two byte selections back and one xor,
 * about 46 instructions per 32-deep step against 16 for Q4_K; it is shared by all the rows
 * of the tile, so tiles are 128 rows high wherever the grid is large enough.
 *
 * Tiling, activation path (three-slot LDS ring filled by buffer_load ... lds from the
 * quantizer's tiled form) and the workgroup-to-XCD mapping are those of gemm_q4k.hip.
 * The weights come from a tile copy in load order (hipq_internal.h, gt_qs / gt_qh / gt_hdr
 * of a Q6_K weight): lane (n, g) of a wavefront owns half g (128 weights) of column n's
 * super-block, eight steps of sixteen weights with one scale each.
 */
#include "gemv_device.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int BN = 128;
constexpr int NT = 256;           /* 4 wavefronts side by side, 32 columns each */
constexpr int QSTAGE = 128 * 128; /* bytes of one stage as the quantizer writes it (128 rows) */

template <int TM> struct Smem6 {
  static constexpr int BM = 32 * TM;
  static constexpr int ASTAGE = BM * 128;
  int8_t a[3][ASTAGE]; /* ring of stages, each [row/32][step 4][lane 64][16] */
  float dA[2][BM];
};
static_assert(sizeof(Smem6<2>) * 3 <= 160 * 1024 && sizeof(Smem6<4>) * 2 <= 160 * 1024,
              "three workgroups of 64 rows or two of 128 rows per CU must fit the 160 KB LDS");

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

struct Src6 {
  rsrc_t qt, dAt;
  rsrc_t wq, wh, whd; /* the wavefront's weight tile: nibbles / high bits / scales (descriptors in scalar
                         registers; a lane's address is its lane offset plus a scalar) */
  int wave, lane;
};
typedef unsigned int u4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16(rsrc_t r, uint32_t voff, uint32_t soff) {
  const u4v v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
  return make_uint4(v[0], v[1], v[2], v[3]);
}
struct WHalf6 { /* this lane's four steps of one 128-deep stage */
  uint4 q[2];   /* per step 8 bytes: weight 2i / 2i+1 of the step's 16 in the low / high nibble of byte i */
  uint4 h;      /* per step 4 bytes: byte i = bits 4-5 of weights 2i, 2i+8, 2i+1, 2i+9 (two bits each, in that order) */
};
__device__ __forceinline__ void load_wh(WHalf6 &W, const Src6 &sr, int sb, int h) {
  W.q[0] = ld16(sr.wq, sr.lane * 16, (uint32_t)(sb * 4 + 2 * h) * 1024);
  W.q[1] = ld16(sr.wq, sr.lane * 16, (uint32_t)(sb * 4 + 2 * h + 1) * 1024);
  W.h = ld16(sr.wh, sr.lane * 16, (uint32_t)(sb * 2 + h) * 1024);
}
template <int TM>
__device__ __forceinline__ void dma_a(const Src6 &sr, Smem6<TM> &sm, int stage, int slot) {
  const uint32_t so = (uint32_t)stage * QSTAGE + sr.wave * (TM * 1024);
  int8_t *l = sm.a[slot] + sr.wave * (TM * 1024);
#pragma unroll
  for (int i = 0; i < TM; ++i) dma16(sr.qt, sr.lane * 16, so + i * 1024, l + i * 1024);
}
/* the rows' scales of a super-block: wavefront 0 (and 1 for 128 rows) copies 64 of them */
template <int TM>
__device__ __forceinline__ void dma_rows(const Src6 &sr, Smem6<TM> &sm, int sb, int buf) {
  if (sr.wave < TM / 2) /* uniform per wavefront */
    dma4(sr.dAt, sr.lane * 4, (uint32_t)sb * (128 * 4) + sr.wave * 256, sm.dA[buf] + sr.wave * 64);
}
/* Loads a wavefront issues at least per stage (wavefronts 2 and 3 copy no scales): what
 * may stay in flight at the stage's barrier. */
template <int TM> struct InFlight6 {
  static constexpr int FIRST = TM + 3;  /* copies of the ring, two nibble loads, the high bits */
  static constexpr int SECOND = TM + 4; /* the same and the next super-block's scales */
};

/* a * b + c in both 16-bit lanes (the compiler's own choice for the expression is a subtract
 * and a multiply) */
__device__ __forceinline__ uint32_t pk_mad(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t r;
  asm("v_pk_mad_i16 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
/* Four 6-bit weights u, one per byte of x, times the step's scale s. In 16-bit lanes
 *     t = u * 4s + (128 - 128 s) = 4 (u - 32) s + 128,     |4 (u - 32) s| <= 16256,
 * so that 4 (u - 32) s = 256 * hi(t) + (lo(t) - 128) with hi the signed high byte of t and
 * lo(t) - 128 = lo(t) ^ 0x80 a signed byte: both operand bytes come out of t by byte
 * selection, no shifts or masks. The two planes then hold four times the product; the
 * factor leaves with the column scale. */
__device__ __forceinline__ void scale_split(uint32_t x, uint32_t s2, uint32_t c2, int &l, int &h) {
  const uint32_t ta = pk_mad(__builtin_amdgcn_perm(x, x, 0x0c020c00u), s2, c2); /* bytes 0 and 2 */
  const uint32_t tb = pk_mad(__builtin_amdgcn_perm(x, x, 0x0c030c01u), s2, c2); /* bytes 1 and 3 */
  l = (int)(__builtin_amdgcn_perm(tb, ta, 0x06020400u) ^ 0x80808080u); /* low bytes: a0 b0 a1 b1 */
  h = (int)__builtin_amdgcn_perm(tb, ta, 0x07030501u);                 /* high bytes */
}

/* four 32-deep steps of one 128-deep stage: H = which half of the lane's eight steps */
template <int H, int TM>
__device__ __forceinline__ void stage_mma(const Smem6<TM> &sm, int slot, const WHalf6 &W, uint2 sc8, int lane,
                                          v16i (&Dl)[TM], v16i (&Dh)[TM]) {
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int8_t *pa = sm.a[0] + slot * Smem6<TM>::ASTAGE + lane * 16;
  v4i a[2][TM];
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) a[0][tm] = *(const v4i *)(pa + (tm * 4) * 1024);
  const uint32_t scw = H ? sc8.y : sc8.x; /* the scales of steps 4H .. 4H+3, one per byte */
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    if (ks + 1 < 4) {
#pragma unroll
      for (int tm = 0; tm < TM; ++tm) a[(ks + 1) & 1][tm] = *(const v4i *)(pa + (tm * 4 + ks + 1) * 1024);
    }
    const uint32_t x0 = ks & 1 ? W.q[ks >> 1].z : W.q[ks >> 1].x, x1 = ks & 1 ? W.q[ks >> 1].w : W.q[ks >> 1].y;
    const uint32_t hb = ks == 0 ? W.h.x : ks == 1 ? W.h.y : ks == 2 ? W.h.z : W.h.w;
    /* four times the scale, sign-extended, in both 16-bit lanes; c2 = 128 - 128 * scale */
    const int s = __builtin_amdgcn_sbfe((int)scw, 8 * ks, 8) << 2;
    const uint32_t s2 = __builtin_amdgcn_perm((uint32_t)s, (uint32_t)s, 0x05040100u);
    const uint32_t c2 = pk_mad(s2, 0xffe0ffe0u, 0x00800080u);
    /* 6-bit weights, one per byte: the even ones (0, 2 .. 14), then the odd ones */
    const uint32_t e0 = (x0 & HIPQ_M4) | ((hb << 4) & 0x30303030u);
    const uint32_t e1 = (x1 & HIPQ_M4) | ((hb << 2) & 0x30303030u);
    const uint32_t o0 = ((x0 >> 4) & HIPQ_M4) | (hb & 0x30303030u);
    const uint32_t o1 = ((x1 >> 4) & HIPQ_M4) | ((hb >> 2) & 0x30303030u);
    int l0, l1, l2, l3, h0, h1, h2, h3;
    scale_split(e0, s2, c2, l0, h0);
    scale_split(e1, s2, c2, l1, h1);
    scale_split(o0, s2, c2, l2, h2);
    scale_split(o1, s2, c2, l3, h3);
    const v4i bl = {l0, l1, l2, l3}, bh = {h0, h1, h2, h3};
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      Dl[tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks & 1][tm], bl, (H == 0 && ks == 0) ? zero16 : Dl[tm], 0, 0, 0);
      Dh[tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks & 1][tm], bh, (H == 0 && ks == 0) ? zero16 : Dh[tm], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <int TM>
__device__ __forceinline__ void epilogue(const Smem6<TM> &sm, int buf, float dcol, int lane, const v16i (&Dl)[TM],
                                         const v16i (&Dh)[TM], float (&acc)[TM][16]) {
  const int g = lane >> 5;
#pragma unroll
  for (int tm = 0; tm < TM; ++tm) {
    const int rbase = tm * 32;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const v4i dv = *(const v4i *)((const int8_t *)sm.dA[buf] + (rbase + 8 * q4 + 4 * g) * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * q4 + e;
        const int I = (Dh[tm][r] << 8) + Dl[tm][r];
        const float tt = dcol * (float)I;
        acc[tm][r] = fmaf(__int_as_float(dv[e]), tt, acc[tm][r]);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(acc[tm][r]));
    __builtin_amdgcn_sched_barrier(0);
  }
}

/* The tile of workgroup blockIdx.x. KSPLIT: its sum over super-blocks sb0 .. sb0 + nsb_part - 1 only
 * (a partial product; the caller adds the parts): everything the loop reads is addressed relative to
 * its first super-block, so the part's first one becomes that by moving the bases. */
template <int TM, bool KSPLIT>
__device__ __forceinline__ void gemm_q6k_tile(const WView &w, const int8_t *__restrict__ qt,
                                              const float *__restrict__ dAt, int M, int mtiles, int ntiles,
                                              float *__restrict__ C, int64_t ldc, int sb0, int nsb_part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem6<TM> &sm = *reinterpret_cast<Smem6<TM> *>(smem_raw);
  constexpr int BM = 32 * TM;
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles, nt = (qd / mtiles) * 8 + xcd;
  if (nt >= ntiles) return; /* uniform per workgroup */
  const int m0 = mt * BM, n0 = nt * BN;
  const int nsb_all = w.K >> 8;
  const int first = KSPLIT ? sb0 : 0;
  const int nsb = KSPLIT ? nsb_part : nsb_all; /* the super-blocks this call walks */
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int i32 = lane & 31;

  Src6 sr;
  /* the quantizer tiles by 128 rows: a 64-row tile is half mt & 1 of quantizer tile mt / 2 */
  const int qt128 = TM == 2 ? mt >> 1 : mt, hrow = TM == 2 ? mt & 1 : 0;
  sr.qt = make_rsrc(qt + ((size_t)qt128 * (2 * nsb_all) + 2 * first) * QSTAGE + hrow * 8192, (uint32_t)(2 * nsb) * QSTAGE);
  sr.dAt = make_rsrc(dAt + ((size_t)qt128 * nsb_all + first) * 128 + hrow * 64, (uint32_t)nsb * 128 * 4);
  /* the copy pads N to 32 rows: a wavefront whose columns start below N has its tile */
  const size_t wt = (size_t)(min(n0 + wave * 32, (int)w.N - 1) >> 5);
  sr.wq = make_rsrc(w.qs + (wt * nsb_all + first) * 4096, (uint32_t)nsb * 4096);
  sr.wh = make_rsrc(w.qh + (wt * nsb_all + first) * 2048, (uint32_t)nsb * 2048);
  sr.whd = make_rsrc(w.hdr + (wt * nsb_all + first) * 1024, (uint32_t)nsb * 1024);
  sr.wave = wave;
  sr.lane = lane;

  v16i Dl[TM], Dh[TM];
  float acc[TM][16];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  WHalf6 Wa, Wb; /* first / second half of a super-block */
  uint4 hd0, hd1;
  load_wh(Wa, sr, 0, 0);
  hd0 = ld16(sr.whd, lane * 16, 0);
  dma_rows(sr, sm, 0, 0);
  dma_a(sr, sm, 0, 0);
  dma_a(sr, sm, 1, 1);
  sync_lds<0>();
  int slot = 0; /* ring slot of the current stage */
  const int nstage = 2 * nsb;
  /* One super-block = two 128-deep stages; each stage first issues what later stages need
   * (the copy of the stage after next into the ring slot read last, the other half's weight
   * bits, once per super-block the next one's row scales and weight scales), then runs its
   * four matrix steps; the barrier at its end waits for the loads issued BEFORE this stage
   * (they retire in order) and leaves this stage's in flight. */
  auto super_block = [&](int sb, const uint4 &hd, uint4 &hdn, int eb) {
    const int sbn = min(sb + 1, nsb - 1);
    const uint2 sc8 = make_uint2(hd.x, hd.y); /* the eight scales of this lane's half */
    const float dcol = 0.25f * hipq_h2f((uint16_t)(hd.z & 0xffff)); /* the planes hold four times the products */
    {
      const int s2 = slot >= 1 ? slot - 1 : 2; /* the slot read last stage */
      dma_a(sr, sm, min(2 * sb + 2, nstage - 1), s2);
      load_wh(Wb, sr, sb, 1);
      stage_mma<0>(sm, slot, Wa, sc8, lane, Dl, Dh);
      slot = slot == 2 ? 0 : slot + 1;
      sync_lds<InFlight6<TM>::FIRST>();
    }
    {
      const int s2 = slot >= 1 ? slot - 1 : 2;
      dma_a(sr, sm, min(2 * sb + 3, nstage - 1), s2);
      load_wh(Wa, sr, sbn, 0);
      hdn = ld16(sr.whd, lane * 16, (uint32_t)sbn * 1024);
      dma_rows(sr, sm, sbn, eb ^ 1);
      stage_mma<1>(sm, slot, Wb, sc8, lane, Dl, Dh);
      slot = slot == 2 ? 0 : slot + 1;
    }
    epilogue(sm, eb, dcol, lane, Dl, Dh, acc);
    sync_lds<InFlight6<TM>::SECOND>();
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

template <int TM>
__global__ __launch_bounds__(NT, TM == 2 ? 3 : 2) void gemm_q6k_kernel(WView w, const int8_t *__restrict__ qt,
                                                                       const float *__restrict__ dAt, int M, int mtiles,
                                                                       int ntiles, float *__restrict__ C, int64_t ldc) {
  gemm_q6k_tile<TM, false>(w, qt, dAt, M, mtiles, ntiles, C, ldc, 0, 0);
}

/* Few tiles (up to 128 rows against a matrix of a few thousand columns make under two hundred
 * workgroups, each walking all of K): blockIdx.y takes a part of K and writes its partial product to
 * part[y]; split_sum6_kernel adds the parts in ascending order. */
__global__ __launch_bounds__(NT, 3) void gemm_q6k_split_kernel(WView w, const int8_t *__restrict__ qt,
                                                               const float *__restrict__ dAt, int M, int mtiles,
                                                               int ntiles, int sb_per_part, float *__restrict__ part,
                                                               int64_t part_stride) {
  const int sb0 = blockIdx.y * sb_per_part;
  gemm_q6k_tile<2, true>(w, qt, dAt, M, mtiles, ntiles, part + (int64_t)blockIdx.y * part_stride, w.N, sb0,
                         min(sb_per_part, (w.K >> 8) - sb0));
}

__global__ __launch_bounds__(256) void split_sum6_kernel(const float *__restrict__ part, int parts, int64_t part_stride,
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

} // namespace

namespace hipq {

template <int TM>
static int launch_tiles6(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc, hipStream_t s) {
  const int mtiles = (M + 32 * TM - 1) / (32 * TM);
  const int ntiles = (int)((w->N + BN - 1) / BN);
  const int ngroups = (ntiles + 7) / 8;
  const unsigned grid = (unsigned)(mtiles * ngroups * 8);
  WView v = wview(w);
  v.qs = w->gt_qs;
  v.qh = w->gt_qh;
  v.hdr = w->gt_hdr;
  hipq::launch_kernel(TM == 2 ? "gemm_q6k_kernel<2>" : "gemm_q6k_kernel<4>", gemm_q6k_kernel<TM>, dim3(grid), dim3(NT), sizeof(Smem6<TM>), s, v, (const int8_t *)qa->qt,
                (const float *)qa->dAt, M, mtiles, ntiles, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* Parts of K for a product whose 64-row tiles would leave most of the chip idle (0: none), and the
 * bytes of partial products they need (the rule of the Q4_K product, gemm_q4k.hip). */
int gemm_q6k_split_parts(const hipq_weight *w, int64_t M) {
  if (w->dtype != HIPQ_Q6_K || !w->gt_base || (w->N & 3)) return 0;
  const int64_t tiles = ((M + 63) / 64) * ((w->N + BN - 1) / BN), nsb = w->K / 256;
  if (tiles > 192 || nsb < 8) return 0;
  int parts = (int)(768 / tiles); /* three workgroups a CU */
  if (parts > 8) parts = 8;
  if (parts > nsb / 4) parts = (int)(nsb / 4);
  return parts >= 2 ? parts : 0;
}
size_t gemm_q6k_split_bytes(const hipq_weight *w, int64_t M) {
  return (size_t)gemm_q6k_split_parts(w, M) * (size_t)M * (size_t)w->N * 4;
}

int launch_gemm_q6k(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc, hipStream_t s,
                    void *partials) {
  if ((M + 127) / 128 != qa->mtiles || qa->K != w->K)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "tiled activations do not match the matmul shape");
  if (!w->gt_base) return fail(HIPQ_ERR_INVALID_ARGUMENT, "the Q6_K prefill product needs the weight's tile copy");
  const int parts = partials ? gemm_q6k_split_parts(w, M) : 0;
  if (parts && !(ldc & 3) && !((uintptr_t)C & 15)) {
    const int nsb = (int)(w->K / 256), per = (nsb + parts - 1) / parts;
    const int mtiles = (M + 63) / 64, ntiles = (int)((w->N + BN - 1) / BN), ngroups = (ntiles + 7) / 8;
    const int64_t stride = (int64_t)M * w->N;
    WView v = wview(w);
    v.qs = w->gt_qs;
    v.qh = w->gt_qh;
    v.hdr = w->gt_hdr;
    hipq::launch_kernel("gemm_q6k_split_kernel", gemm_q6k_split_kernel, dim3((unsigned)(mtiles * ngroups * 8), (unsigned)((nsb + per - 1) / per)),
                  dim3(NT), sizeof(Smem6<2>), s, v, (const int8_t *)qa->qt, (const float *)qa->dAt, M, mtiles, ntiles,
                  per, (float *)partials, stride);
    HIPQ_HIP(hipGetLastError());
    hipq::launch_kernel("split_sum6_kernel", split_sum6_kernel, dim3((unsigned)((stride / 4 + 255) / 256)), dim3(256), 0, s,
                       (const float *)partials, (nsb + per - 1) / per, stride, M, (int)w->N, C, ldc);
    HIPQ_HIP(hipGetLastError());
    return HIPQ_OK;
  }
  /* 128-row tiles halve the expansion per row (the larger part of this kernel's vector work):
   * 862 against 726 TOP/s at 2048 x 12288 x 4096, 835 against 729 at 512 x 151936 x 4096. Two
   * of their workgroups fit a CU instead of three, so they never need more rounds than the
   * 64-row tiles (512 tiles of twice the rows against 768 per round); they lose only where
   * there are too few of them to give every CU one. */
  const int64_t tiles128 = ((int64_t)(M + 127) / 128) * ((w->N + BN - 1) / BN);
  if (M > 64 && tiles128 >= 256) return launch_tiles6<4>(w, qa, M, C, ldc, s);
  return launch_tiles6<2>(w, qa, M, C, ldc, s);
}

} // namespace hipq
