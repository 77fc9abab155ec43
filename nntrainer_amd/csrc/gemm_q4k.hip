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
 * Tiling. A workgroup (4 wavefronts, 2 x 2) owns a 128 x 64 tile of C, each
 * wavefront 64 x 32 (2 MFMA tiles x 2 digit chains). K is walked in stages of
 * 64. Three workgroups share a CU (47 KB of LDS and at most 168 registers each),
 * so one's matrix phase overlaps the others' expansion and epilogue, and the 768
 * tiles of the 512 x 12288 reference shape are all resident at once.
 *  - Activations come from the quantizer already in operand order, 16 KB per
 *    128-row stage (hipq_internal.h, QActTiled), and go from HBM/L2 straight
 *    into LDS with global_load_lds_dwordx4: no registers, no ALU work, and the
 *    ds_read_b128 of a wavefront covers 1 KB of consecutive LDS.
 *  - Weights are read as packed nibbles one super-block ahead (registers) and
 *    expanded into the two digit planes once per workgroup on the way to LDS;
 *    HBM only carries the 4.5-bit form. Plane rows are padded to 80 bytes so
 *    that the 16 lanes of a ds_read_b128 phase hit 16 disjoint 4-bank groups.
 *  - The per-row data of a super-block (bsum parts, d) is copied the same way.
 * Workgroup ids are mapped so that the M-tiles sharing a weight tile run on the
 * same XCD (same L2).
 */
#include "gemv_device.h"

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));

constexpr int BM = 128, BN = 64, KS = 64;
constexpr int NT = 256;         /* 4 wavefronts (2 x 2), 64 x 32 outputs each */
constexpr int STRIDE = KS + 16; /* bytes per staged weight row */
constexpr int ATILE = BM * 128; /* bytes of one 128-deep activation tile as the quantizer writes it */
constexpr int ASTAGE = BM * KS; /* bytes of one 64-deep stage of it */

struct Smem {
  int8_t a[3][ASTAGE]; /* a ring of stages, each [row/32][k/32][k%2][row%32][k%32/2] */
  int8_t blo[2][BN * STRIDE];
  int8_t bhi[2][BN * STRIDE];
  /* per super-block */
  _Float16 amin[BM * 16]; /* per row: 8 low parts, 8 high parts of bsum32_j */
  float dA[BM];
  uint4 colhd[2][BN]; /* per column: the super-block header {d, dmin, scales[12]} */
};
static_assert(sizeof(Smem) * 3 <= 160 * 1024, "three workgroups per CU must fit the 160 KB LDS");

/* per 16-bit half: (two bytes <= 15) * (digit <= 7): no carry between bytes */
__device__ __forceinline__ uint32_t pk_scale(uint32_t x, uint32_t digit2) {
  const v2us r = __builtin_bit_cast(v2us, x) * __builtin_bit_cast(v2us, digit2);
  return __builtin_bit_cast(uint32_t, r);
}

/* 64 lanes x 16 bytes (or x 4 bytes) from global memory to LDS without passing
 * through registers: lane l's bytes land at lds + l * size. lds and soff are
 * uniform. The buffer form is used rather than the global one because the
 * compiler counts buffer loads as ordinary in-order loads; after a global
 * direct-to-LDS load it would wait for ALL loads in flight at the next use of
 * any loaded register, which would drain the weight prefetch. */
typedef __amdgpu_buffer_rsrc_t rsrc_t;
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

/* LDS stores the compiler does not see. It guards every LDS store it knows of
 * that follows a direct-to-LDS copy with a wait for ALL loads in flight, which
 * would drain the weight prefetch at every expansion. These stores never touch
 * a buffer a copy in flight writes; the barrier waits for them (lgkmcnt). */
__device__ __forceinline__ uint32_t lds_addr(const void *p) {
  return (uint32_t)(size_t)(const __attribute__((address_space(3))) void *)p;
}
template <int OFF>
__device__ __forceinline__ void lds_store8(uint32_t addr, uint32_t x, uint32_t y) {
  const v2i v = {(int)x, (int)y};
  asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_store16(uint32_t addr, const uint4 &q) {
  const v4i v = {(int)q.x, (int)q.y, (int)q.z, (int)q.w};
  asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}

/* Everything a thread needs to find its share of the inputs. */
struct Src {
  rsrc_t qt;   /* activation tiles of this M-tile: + tile * ATILE */
  rsrc_t amin; /* + sb * BM * 32 bytes */
  rsrc_t dAt;  /* + sb * BM * 4 bytes */
  const uint8_t *qs, *hdr;
  uint32_t bq; /* byte offset of this thread's 8 weight bytes of stage 0, + sb * 128 + stage * 32 */
  uint32_t hd; /* byte offset of its column's headers, + sb * 16 */
  uint32_t bdst; /* LDS address of its expanded weights relative to a plane buffer */
  int wave, lane;
};

/* stage s4 of super-block sb -> ring slot buf: wavefront w copies rows 32w..32w+31 */
__device__ __forceinline__ void dma_a(const Src &sr, Smem &sm, int sb, int s4, int buf) {
  const uint32_t so = (uint32_t)(sb * 2 + (s4 >> 1)) * ATILE + sr.wave * 4096 + (s4 & 1) * 2048;
  int8_t *l = sm.a[buf] + sr.wave * 2048;
  dma16(sr.qt, sr.lane * 16, so, l);
  dma16(sr.qt, sr.lane * 16, so + 1024, l + 1024);
}

/* per-row data of super-block sb */
__device__ __forceinline__ void dma_rows(const Src &sr, Smem &sm, int sb) {
  dma16(sr.amin, sr.lane * 16, (uint32_t)sb * (BM * 32) + sr.wave * 1024, (char *)sm.amin + sr.wave * 1024);
  if (sr.wave < 2) /* uniform per wavefront */
    dma4(sr.dAt, sr.lane * 4, (uint32_t)sb * (BM * 4) + sr.wave * 256, sm.dA + sr.wave * 64);
}

__device__ __forceinline__ uint2 load_piece(const Src &sr, int sb, int s4) {
  typedef unsigned v2u __attribute__((ext_vector_type(2)));
  const v2u v = __builtin_nontemporal_load((const v2u *)(sr.qs + (sr.bq + (uint32_t)(sb * 128 + s4 * 32))));
  return make_uint2(v[0], v[1]);
}
__device__ __forceinline__ uint4 load_hd(const Src &sr, int sb) {
  return *(const uint4 *)(sr.hdr + (sr.hd + (uint32_t)(sb * 16)));
}

/* Expand this thread's 16 weights of stage S4 (8 bytes: weight 2i / 2i+1 in the low /
 * high nibble of byte i, half a sub-block) into the two digit planes of buffer
 * buf: the even weights are operand bytes of lanes 0-31 of the sub-block's matrix
 * step, the odd ones of lanes 32-63 (the quantizer lays the activations out the
 * same way). */
template <int S4, int BUF, int HDBUF>
struct Expand {
  const uint2 &q;
  const uint4 &hd;
  const Src &sr;
  uint32_t lo, hi, e0, e1, o0, o1;
  static constexpr int LO = offsetof(Smem, blo) + BUF * BN * STRIDE, HI = offsetof(Smem, bhi) + BUF * BN * STRIDE;
  __device__ __forceinline__ Expand(const uint2 &q_, const uint4 &hd_, const Src &sr_) : q(q_), hd(hd_), sr(sr_) {}
  /* The work comes in six parts so that the matrix phase can issue one between
   * every two MFMAs: a wavefront's own vector instructions run in the shadow of
   * its MFMAs, while those of another wavefront mostly wait for them. */
  template <int P>
  __device__ __forceinline__ void part() {
    if (P == 0) {
      const int ksl = (threadIdx.x >> 1) & 1; /* sub-block 2*S4 + ksl */
      /* 6-bit scale of sub-block j: byte j of y for j < 4, else low nibble of byte
       * j-4 of w and bits 6-7 of byte j-4 of y */
      const int sh = 8 * ((2 * S4) & 3) + 8 * ksl;
      const uint32_t sc = S4 < 2 ? ((hd.y >> sh) & 0x3fu)
                                 : (((hd.w >> sh) & 0x0fu) | (((hd.y >> (sh + 6)) & 0x03u) << 4));
      lo = (sc & 7) * 0x00010001u;
      hi = (sc >> 3) * 0x00010001u;
    } else if (P == 1) {
      e0 = q.x & HIPQ_M4, e1 = q.y & HIPQ_M4;
      o0 = (q.x >> 4) & HIPQ_M4, o1 = (q.y >> 4) & HIPQ_M4;
    } else if (P == 2) { /* even weights; the odd ones 16 bytes on */
      lds_store8<LO>(sr.bdst, pk_scale(e0, lo), pk_scale(e1, lo));
    } else if (P == 3) {
      lds_store8<HI>(sr.bdst, pk_scale(e0, hi), pk_scale(e1, hi));
    } else if (P == 4) {
      lds_store8<LO + 16>(sr.bdst, pk_scale(o0, lo), pk_scale(o1, lo));
    } else {
      lds_store8<HI + 16>(sr.bdst, pk_scale(o0, hi), pk_scale(o1, hi));
      if (S4 == 0 && (threadIdx.x & 3) == 0) {
        /* column * 16 from column * STRIDE, recomputed here rather than kept in a
         * register across the loop (the dynamic LDS block starts at address 0) */
        uint32_t x = sr.bdst;
        asm volatile("" : "+v"(x));
        static_assert(STRIDE == 80, "the header address below divides by STRIDE / 16");
        lds_store16<offsetof(Smem, colhd) + HDBUF * BN * 16>((x * 13108u) >> 16, hd);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  __device__ __forceinline__ void all() {
    part<0>(), part<1>(), part<2>(), part<3>(), part<4>(), part<5>();
  }
};

/* Workgroup barrier after this wavefront's LDS stores and after all but the
 * youngest `VM` of its global loads (direct-to-LDS copies included) are done.
 * The generic __syncthreads() would drain every load in flight and throw away
 * the prefetch of the weights. */
template <int VM>
__device__ __forceinline__ void sync_lds() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(VM) : "memory");
}

__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

/* The two 32-deep steps of one stage for the wavefront's 2 x 1 tiles. The second
 * step's weight operands reuse the first step's registers as soon as the MFMAs
 * that read them have issued (operand registers are what keeps three workgroups
 * on a CU). */
template <bool FIRST, class X>
__device__ __forceinline__ void stage_mma(const Smem &sm, int abuf, int bbuf, int wm, int wn, int lane,
                                          v16i (&Dlo)[2], v16i (&Dhi)[2], X &x) {
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int8_t *pa = sm.a[0] + abuf * ASTAGE + (wm * 2) * 2048 + lane * 16;
  const int off = (wn * 32 + (lane & 31)) * STRIDE + (lane >> 5) * 16;
  const int8_t *pl = sm.blo[bbuf] + off, *ph = sm.bhi[bbuf] + off;
  v4i a0 = *(const v4i *)pa, a1 = *(const v4i *)(pa + 2048);
  v4i bl = *(const v4i *)pl, bh = *(const v4i *)ph;
  const v4i c0 = *(const v4i *)(pa + 1024), c1 = *(const v4i *)(pa + 3072);
  __builtin_amdgcn_sched_barrier(0);
  x.template part<0>(); /* covers part of the LDS latency */
  Dlo[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bl, FIRST ? zero16 : Dlo[0], 0, 0, 0);
  x.template part<1>();
  Dlo[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bl, FIRST ? zero16 : Dlo[1], 0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
  bl = *(const v4i *)(pl + 32);
  x.template part<2>();
  Dhi[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bh, FIRST ? zero16 : Dhi[0], 0, 0, 0);
  x.template part<3>();
  Dhi[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bh, FIRST ? zero16 : Dhi[1], 0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
  bh = *(const v4i *)(ph + 32);
  x.template part<4>();
  Dlo[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(c0, bl, Dlo[0], 0, 0, 0);
  x.template part<5>();
  Dlo[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(c1, bl, Dlo[1], 0, 0, 0);
  Dhi[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(c0, bh, Dhi[0], 0, 0, 0);
  Dhi[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(c1, bh, Dhi[1], 0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
}

struct Ctx {
  int wm, wn, i32, g, lane;
};

/* acc += dA * (d * (Dlo + 8 Dhi) - dmin * sum_j m_j bsum_j) for one super-block */
__device__ __forceinline__ void epilogue(const Smem &sm, int buf, const Ctx &c, const v16i (&Dlo)[2],
                                         const v16i (&Dhi)[2], float (&acc)[2][16]) {
  const v16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  /* every compiler-visible LDS access of this kernel is a plain 4 x int vector
   * load: the compiler then tells them apart from the direct-to-LDS copies in
   * flight instead of waiting for all of those before each access */
  const v4i hdv = *(const v4i *)((const int8_t *)sm.colhd[buf] + (c.wn * 32 + c.i32) * 16);
  const uint4 hd = make_uint4((uint32_t)hdv[0], (uint32_t)hdv[1], (uint32_t)hdv[2], (uint32_t)hdv[3]);
  const float dcol = hipq_h2f((uint16_t)(hd.x & 0xffff));
  const float ndmin = -hipq_h2f((uint16_t)(hd.x >> 16));
  const uint32_t mlo = hd.z & 0x3f3f3f3fu;
  const uint32_t mhi = ((hd.w >> 4) & 0x0f0f0f0fu) | (((hd.z >> 6) & 0x03030303u) << 4);
  v8h bmin;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    bmin[j] = (_Float16)(float)((mlo >> (8 * j)) & 0xff);
    bmin[4 + j] = (_Float16)(float)((mhi >> (8 * j)) & 0xff);
  }
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    const int rbase = c.wm * 64 + tm * 32;
    /* lanes 0-31 feed the low parts of bsum, lanes 32-63 the high parts */
    const v8h amin = __builtin_bit_cast(
      v8h, *(const v4i *)((const int8_t *)sm.amin + ((rbase + c.i32) * 16 + c.g * 8) * 2));
    const v16f Sm = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const v4i dv = *(const v4i *)((const int8_t *)sm.dA + (rbase + 8 * q4 + 4 * c.g) * 4);
      const float dA[4] = {__int_as_float(dv[0]), __int_as_float(dv[1]), __int_as_float(dv[2]),
                           __int_as_float(dv[3])};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * q4 + e;
        const int I = (Dhi[tm][r] << 3) + Dlo[tm][r];
        float tt = dcol * (float)I;
        tt = fmaf(ndmin, Sm[r], tt);
        acc[tm][r] = fmaf(dA[e], tt, acc[tm][r]);
      }
    }
    /* Pin the sums here. Left alone the compiler sinks this arithmetic past the
     * barrier and keeps the integer tiles alive into the next super-block. */
#pragma unroll
    for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(acc[tm][r]));
    __builtin_amdgcn_sched_barrier(0);
  }
}

/* One stage S4 of super-block sb. On entry ring slot `ar` holds this stage's
 * activations (copied two stages ago) and the plane buffers S4 & 1 its expanded
 * weights. The stage runs its matrix steps and, between them, expands the NEXT
 * stage's weights (loaded one super-block ago) into the other plane buffers;
 * then it issues the copy of the activation stage after next and reloads the
 * freed weight registers with the same stage of the next super-block. The
 * hardware retires loads in issue order: the barrier waits for the copies of
 * the previous stage (needed next) and leaves this stage's in flight. */
template <int S4, int EB>
__device__ __forceinline__ void stage(Smem &sm, const Src &sr, const Ctx &c, int sb, int nsb, int &ar,
                                      uint2 (&q)[4], const uint4 &hdc, uint4 &hdn, v16i (&Dlo)[2],
                                      v16i (&Dhi)[2], float (&acc)[2][16]) {
  constexpr int N4 = (S4 + 1) & 3; /* the stage expanded now */
  const int sbn = min(sb + 1, nsb - 1), sbnn = min(sb + 2, nsb - 1);
  /* stage 3 expands stage 0 of the next super-block, and stores its headers */
  Expand<N4, (S4 + 1) & 1, (S4 < 3 ? EB : EB ^ 1)> x(q[N4], S4 < 3 ? hdc : hdn, sr);
  if (S4 == 0)
    stage_mma<true>(sm, ar, 0, c.wm, c.wn, c.lane, Dlo, Dhi, x);
  else
    stage_mma<false>(sm, ar, S4 & 1, c.wm, c.wn, c.lane, Dlo, Dhi, x);
  const int a2 = ar == 0 ? 2 : ar - 1; /* the slot read last stage: ar, ar + 1, a2 rotate */
  if (S4 < 2)
    dma_a(sr, sm, sb, S4 + 2, a2);
  else
    dma_a(sr, sm, sbn, S4 - 2, a2);
  if (S4 == 0) dma_rows(sr, sm, sb); /* last read by the epilogue of sb - 1, next by this one's */
  q[N4] = load_piece(sr, S4 < 3 ? sbn : sbnn, N4);
  if (S4 == 0) hdn = load_hd(sr, sbn);
  __builtin_amdgcn_sched_barrier(0);
  if (S4 == 3) epilogue(sm, EB, c, Dlo, Dhi, acc);
  ar = ar == 2 ? 0 : ar + 1;
  /* everything issued before this stage has landed; this stage's 3 (5 or 6 in
   * stage 0) copies and loads stay in flight */
  sync_lds<(S4 == 0 ? 5 : 3)>();
}

template <int EB>
__device__ __forceinline__ void super_block(Smem &sm, const Src &sr, const Ctx &c, int sb, int nsb,
                                            int &ar, uint2 (&q)[4], uint4 &hdc, uint4 &hdn,
                                            v16i (&Dlo)[2], v16i (&Dhi)[2], float (&acc)[2][16]) {
  stage<0, EB>(sm, sr, c, sb, nsb, ar, q, hdc, hdn, Dlo, Dhi, acc);
  stage<1, EB>(sm, sr, c, sb, nsb, ar, q, hdc, hdn, Dlo, Dhi, acc);
  stage<2, EB>(sm, sr, c, sb, nsb, ar, q, hdc, hdn, Dlo, Dhi, acc);
  stage<3, EB>(sm, sr, c, sb, nsb, ar, q, hdc, hdn, Dlo, Dhi, acc);
}

__global__ __launch_bounds__(NT, 3) void gemm_q4k_kernel(WView w, const int8_t *__restrict__ qt,
                                                         const uint16_t *__restrict__ amin,
                                                         const float *__restrict__ dAt, int M,
                                                         int mtiles, int ntiles,
                                                         float *__restrict__ C, int64_t ldc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem &sm = *reinterpret_cast<Smem *>(smem_raw);
  if (lds_addr(smem_raw) != 0) __builtin_trap(); /* folds away: no static LDS in this kernel */
  /* workgroup id -> tile: the M-tiles of one weight tile share id % 8 (one XCD) */
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles, nt = (qd / mtiles) * 8 + xcd;
  if (nt >= ntiles) return; /* uniform per workgroup */
  const int m0 = mt * BM, n0 = nt * BN;
  const int nsb = w.K >> 8;
  Ctx c;
  c.lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  c.wm = wave >> 1;
  c.wn = wave & 1;
  c.i32 = c.lane & 31;
  c.g = c.lane >> 5;

  Src sr;
  sr.qt = make_rsrc(qt + (size_t)mt * (2 * nsb) * ATILE, (uint32_t)(2 * nsb) * ATILE);
  sr.amin = make_rsrc(amin + (size_t)mt * nsb * BM * 16, (uint32_t)nsb * BM * 32);
  sr.dAt = make_rsrc(dAt + (size_t)mt * nsb * BM, (uint32_t)nsb * BM * 4);
  sr.qs = w.qs;
  sr.hdr = w.hdr;
  {
    const int t = threadIdx.x;
    const uint32_t n = (uint32_t)min(n0 + (t >> 2), w.N - 1); /* columns past N are never stored */
    sr.bq = n * (uint32_t)(w.K >> 1) + (t & 3) * 8;
    sr.hd = n * (uint32_t)nsb * 16;
    sr.bdst = (t >> 2) * STRIDE + ((t & 3) >> 1) * 32 + (t & 1) * 8;
  }
  sr.wave = wave;
  sr.lane = c.lane;

  v16i Dlo[2], Dhi[2];
  float acc[2][16];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  /* prologue: stage (0, 0) into the buffers 0, weights of super-block 0 into registers */
  uint2 q[4];
  uint4 hd0, hd1;
  hd0 = load_hd(sr, 0);
#pragma unroll
  for (int j = 0; j < 4; ++j) q[j] = load_piece(sr, 0, j);
  Expand<0, 0, 0>(q[0], hd0, sr).all();
  dma_a(sr, sm, 0, 0, 0);
  dma_a(sr, sm, 0, 1, 1);
  q[0] = load_piece(sr, min(1, nsb - 1), 0);
  sync_lds<0>();

  int ar = 0; /* ring slot of the current activation stage */
  int sb = 0;
  for (; sb + 1 < nsb; sb += 2) {
    super_block<0>(sm, sr, c, sb, nsb, ar, q, hd0, hd1, Dlo, Dhi, acc);
    super_block<1>(sm, sr, c, sb + 1, nsb, ar, q, hd1, hd0, Dlo, Dhi, acc);
  }
  if (sb < nsb) super_block<0>(sm, sr, c, sb, nsb, ar, q, hd0, hd1, Dlo, Dhi, acc);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); /* no copy may outlive the workgroup's LDS */

  const int n = n0 + c.wn * 32 + c.i32;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + c.wm * 64 + tm * 32 + acc_row(r, c.lane);
      if (m < M && n < w.N) C[(int64_t)m * ldc + n] = acc[tm][r];
    }
}

} // namespace

namespace hipq {

int launch_gemm_q4k(const hipq_weight *w, const QActTiled *qa, int M, float *C, int64_t ldc,
                    hipStream_t s) {
  const int mtiles = (M + BM - 1) / BM;
  if (mtiles != qa->mtiles || qa->K != w->K)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "tiled activations do not match the matmul shape");
  const int ntiles = (int)((w->N + BN - 1) / BN);
  const int ngroups = (ntiles + 7) / 8;
  const unsigned grid = (unsigned)(mtiles * ngroups * 8);
  hipLaunchKernelGGL(gemm_q4k_kernel, dim3(grid), dim3(NT), sizeof(Smem), s, wview(w), qa->qt, qa->amin,
                     qa->dAt, M, mtiles, ntiles, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
