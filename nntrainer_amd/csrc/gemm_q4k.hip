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
 * 128. Two workgroups share a CU (80 KB of LDS and at most 256 registers each),
 * so one's matrix phase overlaps the other's expansion and epilogue.
 *  - Activations come from the quantizer already in operand order, 16 KB per
 *    128-row stage (hipq_internal.h, QActTiled), and go from HBM/L2 straight
 *    into LDS with global_load_lds_dwordx4: no registers, no ALU work, and the
 *    ds_read_b128 of a wavefront covers 1 KB of consecutive LDS.
 *  - Weights are read as packed nibbles two super-blocks ahead (registers) and
 *    expanded into the two digit planes once per workgroup on the way to LDS;
 *    HBM only carries the 4.5-bit form. Plane rows are padded to 144 bytes so
 *    that the 16 lanes of a ds_read_b128 phase hit 16 disjoint 4-bank groups.
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

constexpr int BM = 128, BN = 64, KS = 128;
constexpr int NT = 256;         /* 4 wavefronts (2 x 2), 64 x 32 outputs each */
constexpr int STRIDE = KS + 16; /* bytes per staged weight row */
constexpr int ATILE = BM * KS;  /* bytes of one activation stage */

struct Smem {
  int8_t a[2][ATILE]; /* [row/32][k/32][k%32/16][row%32][16] */
  int8_t blo[2][BN * STRIDE];
  int8_t bhi[2][BN * STRIDE];
  /* per super-block, double-buffered */
  _Float16 amin[2][BM * 16]; /* per row: 8 low parts, 8 high parts of bsum32_j */
  float dA[2][BM];
  uint4 colhd[2][BN]; /* per column: the super-block header {d, dmin, scales[12]} */
};
static_assert(sizeof(Smem) <= 80 * 1024, "two workgroups per CU must fit the 160 KB LDS");

struct BBlock { /* one super-block of weights: 64 columns x 128 bytes + headers */
  uint4 q0, q1; /* the 16 bytes this thread expands in stage 0 and in stage 1 */
  uint4 hd;
};

/* per 16-bit half: (two bytes <= 15) * (digit <= 7): no carry between bytes */
__device__ __forceinline__ uint32_t pk_scale(uint32_t x, uint32_t digit2) {
  const v2us r = __builtin_bit_cast(v2us, x) * __builtin_bit_cast(v2us, digit2);
  return __builtin_bit_cast(uint32_t, r);
}

/* 64 lanes x 16 bytes (or x 4 bytes) from global memory to LDS without passing
 * through registers: lane l's bytes land at lds + l * size. lds is uniform. */
__device__ __forceinline__ void dma16(const void *gptr_lane, void *lds_wave) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gptr_lane,
                                   (__attribute__((address_space(3))) void *)lds_wave, 16, 0, 0);
}
__device__ __forceinline__ void dma4(const void *gptr_lane, void *lds_wave) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gptr_lane,
                                   (__attribute__((address_space(3))) void *)lds_wave, 4, 0, 0);
}

/* Everything a thread needs to find its share of the inputs. */
struct Src {
  const int8_t *qt;     /* activation stages of this M-tile, + stage * ATILE, + lane part */
  const uint16_t *amin; /* + sb * BM * 16 halfs */
  const float *dAt;     /* + sb * BM */
  const uint8_t *qs, *hdr;
  uint32_t bq; /* byte offset of this thread's weight bytes, + sb * 128 (+ 64) */
  uint32_t hd; /* byte offset of its column's headers, + sb * 16 */
  int wave, lane;
};

/* stage s of the activations -> LDS buffer buf: wavefront w copies rows 32w..32w+31 */
__device__ __forceinline__ void dma_a(const Src &sr, Smem &sm, int s, int buf) {
  const int8_t *g = sr.qt + (size_t)s * ATILE + sr.wave * 4096 + sr.lane * 16;
  int8_t *l = sm.a[buf] + sr.wave * 4096;
#pragma unroll
  for (int c = 0; c < 4; ++c) dma16(g + c * 1024, l + c * 1024);
}

/* per-row data of super-block sb -> LDS buffer buf */
__device__ __forceinline__ void dma_rows(const Src &sr, Smem &sm, int sb, int buf) {
  dma16((const char *)(sr.amin + (size_t)sb * BM * 16) + sr.wave * 1024 + sr.lane * 16,
        (char *)sm.amin[buf] + sr.wave * 1024);
  if (sr.wave < 2) /* uniform per wavefront */
    dma4(sr.dAt + (size_t)sb * BM + sr.wave * 64 + sr.lane, sm.dA[buf] + sr.wave * 64);
}

__device__ __forceinline__ void load_b(BBlock &b, const Src &sr, int sb) {
  b.q0 = hipq_ld_stream((const uint4 *)(sr.qs + (sr.bq + (uint32_t)(sb * 128))));
  b.q1 = hipq_ld_stream((const uint4 *)(sr.qs + (sr.bq + (uint32_t)(sb * 128 + 64))));
  b.hd = *(const uint4 *)(sr.hdr + (sr.hd + (uint32_t)(sb * 16)));
}

/* Expand this thread's 32 weights of stage H into the two digit planes. Its 16
 * bytes are ONE sub-block (weight 2i / 2i+1 in the low / high nibble of byte i),
 * i.e. one 32-deep matrix step of its column: the even weights become the 16
 * operand bytes of lanes 0-31 of that step, the odd ones those of lanes 32-63
 * (the quantizer lays the activations out the same way). */
template <int H>
__device__ __forceinline__ void store_b(const BBlock &b, Smem &sm, int hdbuf) {
  const int t = threadIdx.x;
  const int row = t >> 2, ks = t & 3; /* sub-block 4*H + ks of the super-block */
  const uint4 hd = b.hd;
  /* 6-bit scale of sub-block j: byte j of y for j < 4, else low nibble of byte
   * j of w and bits 6-7 of byte j-4 of y */
  const int sh = 8 * ks;
  const uint32_t sc = H == 0 ? ((hd.y >> sh) & 0x3fu)
                             : (((hd.w >> sh) & 0x0fu) | (((hd.y >> (sh + 6)) & 0x03u) << 4));
  const uint32_t lo = (sc & 7) * 0x00010001u, hi = (sc >> 3) * 0x00010001u;
  const uint4 q = H == 0 ? b.q0 : b.q1;
  const uint32_t E[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
  const uint32_t O[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                         (q.w >> 4) & HIPQ_M4};
  const int d0 = row * STRIDE + ks * 32; /* even weights; the odd ones 16 bytes on */
  auto put = [](int8_t *dst, const uint32_t (&v)[4], uint32_t digit2) {
    *(v4i *)dst = v4i{(int)pk_scale(v[0], digit2), (int)pk_scale(v[1], digit2),
                      (int)pk_scale(v[2], digit2), (int)pk_scale(v[3], digit2)};
  };
  put(sm.blo[H] + d0, E, lo);
  put(sm.bhi[H] + d0, E, hi);
  put(sm.blo[H] + d0 + 16, O, lo);
  put(sm.bhi[H] + d0 + 16, O, hi);
  if (H == 0 && ks == 0)
    *(v4i *)((int8_t *)sm.colhd[hdbuf] + row * 16) = v4i{(int)hd.x, (int)hd.y, (int)hd.z, (int)hd.w};
}

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

/* Operands of one 32-deep step of the wavefront's 2 x 1 tiles. */
struct Ops {
  v4i a0, a1, bl, bh;
};
__device__ __forceinline__ void read_ops(Ops &o, const Smem &sm, int buf, int ks, int wm, int wn,
                                         int lane) {
  const int8_t *pa = sm.a[buf] + ((wm * 2) * 4 + ks) * 1024 + lane * 16;
  o.a0 = *(const v4i *)pa;
  o.a1 = *(const v4i *)(pa + 4096);
  const int off = (wn * 32 + (lane & 31)) * STRIDE + ks * 32 + (lane >> 5) * 16;
  o.bl = *(const v4i *)(sm.blo[buf] + off);
  o.bh = *(const v4i *)(sm.bhi[buf] + off);
}
template <bool FIRST>
__device__ __forceinline__ void mma_ops(const Ops &o, v16i (&Dlo)[2], v16i (&Dhi)[2]) {
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  Dlo[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a0, o.bl, FIRST ? zero16 : Dlo[0], 0, 0, 0);
  Dhi[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a0, o.bh, FIRST ? zero16 : Dhi[0], 0, 0, 0);
  Dlo[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a1, o.bl, FIRST ? zero16 : Dlo[1], 0, 0, 0);
  Dhi[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a1, o.bh, FIRST ? zero16 : Dhi[1], 0, 0, 0);
}

/* The four 32-deep steps of one stage; the operands of step k+1 are read from
 * LDS while the matrix core works on step k. */
template <bool FIRST>
__device__ __forceinline__ void stage_mma(const Smem &sm, int buf, int wm, int wn, int lane,
                                          v16i (&Dlo)[2], v16i (&Dhi)[2]) {
  Ops o0, o1;
  /* the matrix phase goes first when both wavefronts of a SIMD want to issue:
   * the other workgroup's vector work then fills the gaps between MFMAs */
  __builtin_amdgcn_s_setprio(2);
  read_ops(o0, sm, buf, 0, wm, wn, lane);
  read_ops(o1, sm, buf, 1, wm, wn, lane);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<FIRST>(o0, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  read_ops(o0, sm, buf, 2, wm, wn, lane);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o1, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  read_ops(o1, sm, buf, 3, wm, wn, lane);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o0, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o1, Dlo, Dhi);
  __builtin_amdgcn_s_setprio(0);
  __builtin_amdgcn_sched_barrier(0);
}

struct Ctx {
  int wm, wn, i32, g, lane;
};

/* acc += dA * (d * (Dlo + 8 Dhi) - dmin * sum_j m_j bsum_j) for one super-block */
__device__ __forceinline__ void epilogue(const Smem &sm, int buf, const Ctx &c, const v16i (&Dlo)[2],
                                         const v16i (&Dhi)[2], float (&acc)[2][16]) {
  const v16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  /* every LDS access of this kernel is a plain 4 x int vector: the compiler then
   * tells them apart from the direct-to-LDS copies in flight instead of waiting
   * for all of those before each access */
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
      v8h, *(const v4i *)((const int8_t *)sm.amin[buf] + ((rbase + c.i32) * 16 + c.g * 8) * 2));
    const v16f Sm = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const v4i dv = *(const v4i *)((const int8_t *)sm.dA[buf] + (rbase + 8 * q4 + 4 * c.g) * 4);
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

/* One super-block sb (eb = sb & 1 selects its row/column data buffers).
 * On entry LDS holds activation stage (sb, 0) in a[0], the digit planes of
 * stage (sb, 0) in blo/bhi[0], the row data and headers of sb in buffer eb;
 * registers hold the packed weights of sb (bcur) and sb + 1 (bnext).
 * The hardware retires loads in issue order, so each wait names how many
 * younger loads may stay in flight: the weight prefetch (HBM, two super-blocks
 * ahead) is always issued after the copies that are needed first. */
template <int EB>
__device__ __forceinline__ void super_block(Smem &sm, const Src &sr, const Ctx &c, int sb, int nsb,
                                            BBlock &bcur, const BBlock &bnext, v16i (&Dlo)[2],
                                            v16i (&Dhi)[2], float (&acc)[2][16]) {
  const int sb1 = min(sb + 1, nsb - 1), sb2 = min(sb + 2, nsb - 1);
  dma_rows(sr, sm, sb1, EB ^ 1); /* last read by the epilogue of sb - 1 */
  dma_a(sr, sm, sb * 2 + 1, 1);  /* last read by the second stage of sb - 1 */
  __builtin_amdgcn_sched_barrier(0);
  stage_mma<true>(sm, 0, c.wm, c.wn, c.lane, Dlo, Dhi);
  store_b<1>(bcur, sm, 0);
  sync_lds<0>(); /* a[1], the planes of stage 1 and the row data of sb + 1 are in place */
  /* The compiler guards every LDS store that follows a direct-to-LDS copy with a
   * wait for all loads in flight, so the stores go where nothing is in flight:
   * right after the barrier, before the next copies and loads are issued. */
  store_b<0>(bnext, sm, EB ^ 1); /* planes and headers of stage (sb + 1, 0) */
  __builtin_amdgcn_sched_barrier(0);
  dma_a(sr, sm, sb1 * 2, 0);
  load_b(bcur, sr, sb2); /* bcur's registers are free: they become the weights of sb + 2 */
  __builtin_amdgcn_sched_barrier(0);
  stage_mma<false>(sm, 1, c.wm, c.wn, c.lane, Dlo, Dhi);
  epilogue(sm, EB, c, Dlo, Dhi, acc);
  sync_lds<3>(); /* a[0] has landed; the three weight loads stay in flight */
}

__global__ __launch_bounds__(NT, 2) void gemm_q4k_kernel(WView w, const int8_t *__restrict__ qt,
                                                         const uint16_t *__restrict__ amin,
                                                         const float *__restrict__ dAt, int M,
                                                         int mtiles, int ntiles,
                                                         float *__restrict__ C, int64_t ldc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem &sm = *reinterpret_cast<Smem *>(smem_raw);
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
  sr.qt = qt + (size_t)mt * (2 * nsb) * ATILE;
  sr.amin = amin + (size_t)mt * nsb * BM * 16;
  sr.dAt = dAt + (size_t)mt * nsb * BM;
  sr.qs = w.qs;
  sr.hdr = w.hdr;
  {
    const int t = threadIdx.x;
    const uint32_t n = (uint32_t)min(n0 + (t >> 2), w.N - 1); /* columns past N are never stored */
    sr.bq = n * (uint32_t)(w.K >> 1) + (t & 3) * 16;
    sr.hd = n * (uint32_t)nsb * 16;
  }
  sr.wave = wave;
  sr.lane = c.lane;

  v16i Dlo[2], Dhi[2];
  float acc[2][16];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  BBlock b0, b1;
  dma_rows(sr, sm, 0, 0);
  dma_a(sr, sm, 0, 0);
  load_b(b0, sr, 0);
  load_b(b1, sr, min(1, nsb - 1));
  store_b<0>(b0, sm, 0);
  sync_lds<0>();

  int sb = 0;
  for (; sb + 1 < nsb; sb += 2) {
    super_block<0>(sm, sr, c, sb, nsb, b0, b1, Dlo, Dhi, acc);
    super_block<1>(sm, sr, c, sb + 1, nsb, b1, b0, Dlo, Dhi, acc);
  }
  if (sb < nsb) super_block<0>(sm, sr, c, sb, nsb, b0, b1, Dlo, Dhi, acc);
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
  static bool lds_opt_in = false;
  if (!lds_opt_in) {
    HIPQ_HIP(hipFuncSetAttribute((const void *)gemm_q4k_kernel,
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem)));
    lds_opt_in = true;
  }
  hipLaunchKernelGGL(gemm_q4k_kernel, dim3(grid), dim3(NT), sizeof(Smem), s, wview(w), qa->qt, qa->amin,
                     qa->dAt, M, mtiles, ntiles, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
