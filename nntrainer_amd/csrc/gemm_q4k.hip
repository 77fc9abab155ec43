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
 * Tiling. A workgroup (4 wavefronts, 2 x 2) owns a 128 x 128 tile of C.
 * K is walked in stages of 128; per stage the int8 activations and the two
 * digit planes of the weights (expanded from nibbles once per workgroup, on the
 * way from HBM to LDS; HBM only carries the packed 4.5-bit form) sit in LDS,
 * double-buffered, rows padded to 144 bytes so that the 16 lanes of a
 * ds_read_b128 phase hit 16 disjoint 4-bank groups. Each wavefront computes
 * 2 x 2 MFMA tiles (64 x 64). Workgroup ids are mapped so that the M-tiles
 * sharing a weight tile run on the same XCD (same L2).
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
constexpr int STRIDE = KS + 16; /* bytes per staged row */

struct Smem {
  int8_t a[2][BM * STRIDE];
  int8_t blo[2][BN * STRIDE];
  int8_t bhi[2][BN * STRIDE];
  /* per super-block, single-buffered (a barrier separates readers and writer) */
  _Float16 amin[BM * 16]; /* per row: 8 low parts, 8 high parts of bsum32_j */
  float dA[BM];
  uint4 colhd[BN]; /* per column: the super-block header {d, dmin, scales[12]} */
};
static_assert(sizeof(Smem) <= 80 * 1024, "two workgroups per CU must fit the 160 KB LDS");

/* Registers of one workgroup thread between the global loads and the LDS. */
struct AStage { /* one 128-deep stage of activations: 128 rows x 128 bytes */
  v4i a0, a1, a2, a3; /* plain vectors: struct copies would stay in scratch memory */
};
struct BBlock { /* one super-block of weights: 64 columns x 128 bytes + headers */
  uint4 q0, q1; /* the 16 bytes this thread expands in stage 0 and in stage 1 */
  uint4 hd;
};
struct RowBlock { /* per-row data of one super-block (threads 0..127) */
  uint4 bs0 = {0, 0, 0, 0}, bs1 = {0, 0, 0, 0};
  float dA = 0.f;
};

/* per 16-bit half: (two bytes <= 15) * (digit <= 7): no carry between bytes */
__device__ __forceinline__ uint32_t pk_scale(uint32_t x, uint32_t digit2) {
  const v2us r = __builtin_bit_cast(v2us, x) * __builtin_bit_cast(v2us, digit2);
  return __builtin_bit_cast(uint32_t, r);
}

/* Per-thread constant parts of the addresses. Rows past the end of the
 * matrices are clamped (their results are never stored), so no load sits under
 * a lane-dependent branch and the hardware counters wait for each one exactly. */
struct Addr { /* byte offsets from the (uniform) plane pointers; planes are < 4 GiB */
  const int8_t *q;
  const uint8_t *qs, *hdr;
  const int16_t *bsum;
  const float *d;
  uint32_t a[4]; /* + sb * 256 + h * 128 */
  uint32_t bq;   /* + sb * 128 + h * 64 */
  uint32_t hd;   /* + sb * 16 */
  uint32_t bs;   /* + sb * 32 */
  uint32_t dA;   /* + sb * 4 */
};

__device__ __forceinline__ Addr make_addr(const WView &w, const QView &qa, int M, int m0, int n0) {
  const int t = threadIdx.x;
  const int nsb = w.K >> 8;
  Addr ad;
  ad.q = qa.q;
  ad.qs = w.qs;
  ad.hdr = w.hdr;
  ad.bsum = qa.bsum;
  ad.d = qa.d;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = it * NT + t;
    const int row = idx >> 3, c16 = idx & 7;
    ad.a[it] = (uint32_t)min(m0 + row, M - 1) * (uint32_t)qa.K + c16 * 16;
  }
  const uint32_t n = (uint32_t)min(n0 + (t >> 2), w.N - 1);
  ad.bq = n * (uint32_t)(w.K >> 1) + (t & 3) * 16;
  ad.hd = n * (uint32_t)nsb * 16;
  const uint32_t m = (uint32_t)min(m0 + (t & (BM - 1)), M - 1);
  ad.bs = m * (uint32_t)(qa.K >> 4) * 2;
  ad.dA = m * (uint32_t)nsb * 4;
  return ad;
}

__device__ __forceinline__ void load_a(AStage &st, const Addr &ad, int sb, int h) {
  const uint32_t k0 = (uint32_t)(sb * 256 + h * 128);
  st.a0 = *(const v4i *)(ad.q + (ad.a[0] + k0));
  st.a1 = *(const v4i *)(ad.q + (ad.a[1] + k0));
  st.a2 = *(const v4i *)(ad.q + (ad.a[2] + k0));
  st.a3 = *(const v4i *)(ad.q + (ad.a[3] + k0));
}
__device__ __forceinline__ void load_b(BBlock &b, const Addr &ad, int sb) {
  b.q0 = hipq_ld_stream((const uint4 *)(ad.qs + (ad.bq + (uint32_t)(sb * 128))));
  b.q1 = hipq_ld_stream((const uint4 *)(ad.qs + (ad.bq + (uint32_t)(sb * 128 + 64))));
  b.hd = *(const uint4 *)(ad.hdr + (ad.hd + (uint32_t)(sb * 16)));
}
__device__ __forceinline__ void load_row(RowBlock &r, const Addr &ad, int sb) {
  /* whole wavefronts 0 and 1 own the 128 rows; the branch is uniform per wavefront */
  if (__builtin_amdgcn_readfirstlane((int)threadIdx.x) >= BM) return;
  const uint4 *bp = (const uint4 *)((const char *)ad.bsum + (ad.bs + (uint32_t)(sb * 32)));
  r.bs0 = bp[0];
  r.bs1 = bp[1];
  r.dA = *(const float *)((const char *)ad.d + (ad.dA + (uint32_t)(sb * 4)));
}

__device__ __forceinline__ void store_a(const AStage &st, Smem &sm, int buf) {
  const int t = threadIdx.x;
  /* thread t owns 16 bytes of rows t/8, t/8 + 32, t/8 + 64, t/8 + 96 */
  int8_t *p = sm.a[buf] + (t >> 3) * STRIDE + (t & 7) * 16;
  *(v4i *)(p) = st.a0;
  *(v4i *)(p + 32 * STRIDE) = st.a1;
  *(v4i *)(p + 64 * STRIDE) = st.a2;
  *(v4i *)(p + 96 * STRIDE) = st.a3;
}

/* Expand this thread's 32 weights of stage h into the two digit planes. */
template <int H>
__device__ __forceinline__ void store_b(const BBlock &b, Smem &sm) {
  const int t = threadIdx.x;
  const int row = t >> 2, c16 = t & 3;
  const int p = c16 >> 1, hh = c16 & 1; /* sub-block pair 2*H + p of the super-block */
  const uint4 hd = b.hd;
  const int sh = 16 * p;
  const uint32_t y = hd.y >> sh, ww = hd.w >> sh;
  /* scales of sub-blocks 4..7 are spread over two header words */
  const uint32_t scw = H == 0 ? (y & 0x3f3fu) : ((ww & 0x0f0fu) | (((y >> 6) & 0x0303u) << 4));
  const uint32_t sc0 = scw & 0xff, sc1 = scw >> 8;
  const uint32_t lo0 = (sc0 & 7) * 0x00010001u, hi0 = (sc0 >> 3) * 0x00010001u;
  const uint32_t lo1 = (sc1 & 7) * 0x00010001u, hi1 = (sc1 >> 3) * 0x00010001u;
  const uint4 q = H == 0 ? b.q0 : b.q1;
  const uint32_t L[4] = {q.x & HIPQ_M4, q.y & HIPQ_M4, q.z & HIPQ_M4, q.w & HIPQ_M4};
  const uint32_t Hn[4] = {(q.x >> 4) & HIPQ_M4, (q.y >> 4) & HIPQ_M4, (q.z >> 4) & HIPQ_M4,
                          (q.w >> 4) & HIPQ_M4};
  const int d0 = row * STRIDE + (2 * p) * 32 + hh * 16; /* even sub-block: low nibbles */
  const int d1 = d0 + 32;                               /* odd sub-block: high nibbles */
  *(uint4 *)(sm.blo[H] + d0) =
    make_uint4(pk_scale(L[0], lo0), pk_scale(L[1], lo0), pk_scale(L[2], lo0), pk_scale(L[3], lo0));
  *(uint4 *)(sm.bhi[H] + d0) =
    make_uint4(pk_scale(L[0], hi0), pk_scale(L[1], hi0), pk_scale(L[2], hi0), pk_scale(L[3], hi0));
  *(uint4 *)(sm.blo[H] + d1) = make_uint4(pk_scale(Hn[0], lo1), pk_scale(Hn[1], lo1),
                                          pk_scale(Hn[2], lo1), pk_scale(Hn[3], lo1));
  *(uint4 *)(sm.bhi[H] + d1) = make_uint4(pk_scale(Hn[0], hi1), pk_scale(Hn[1], hi1),
                                          pk_scale(Hn[2], hi1), pk_scale(Hn[3], hi1));
  if (H == 0 && c16 == 0) sm.colhd[row] = hd;
}

__device__ __forceinline__ void store_row(const RowBlock &rb, Smem &sm) {
  const int t = threadIdx.x;
  if (__builtin_amdgcn_readfirstlane(t) < BM) {
    const uint32_t wds[8] = {rb.bs0.x, rb.bs0.y, rb.bs0.z, rb.bs0.w,
                             rb.bs1.x, rb.bs1.y, rb.bs1.z, rb.bs1.w};
    v8h vlo, vhi;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int bs = (int)(int16_t)(wds[j] & 0xffff) + ((int)wds[j] >> 16); /* |bs| <= 4064 */
      const int l6 = bs & 63;
      vlo[j] = (_Float16)(float)l6;        /* 0..63 */
      vhi[j] = (_Float16)(float)(bs - l6); /* multiple of 64, 7 significant bits */
    }
    *(v8h *)(sm.amin + t * 16) = vlo;
    *(v8h *)(sm.amin + t * 16 + 8) = vhi;
    sm.dA[t] = rb.dA;
  }
}

/* Workgroup barrier that only waits for this wavefront's LDS traffic. The
 * generic __syncthreads() also drains the global loads in flight, which would
 * throw away the prefetch of the next stages. */
__device__ __forceinline__ void sync_lds() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ int acc_row(int r, int lane) {
  return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

/* Operands of one 32-deep step of the wavefront's 2 x 1 tiles. */
struct Ops {
  v4i a0, a1, bl, bh;
};
__device__ __forceinline__ void read_ops(Ops &o, const Smem &sm, int buf, int ks, int wm, int wn,
                                         int i32, int g) {
  const int8_t *pa = sm.a[buf] + (wm * 64 + i32) * STRIDE + ks * 32 + g * 16;
  o.a0 = *(const v4i *)pa;
  o.a1 = *(const v4i *)(pa + 32 * STRIDE);
  const int off = (wn * 32 + i32) * STRIDE + ks * 32 + g * 16;
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
__device__ __forceinline__ void stage_mma(const Smem &sm, int buf, int wm, int wn, int i32, int g,
                                          v16i (&Dlo)[2], v16i (&Dhi)[2]) {
  Ops o0, o1;
  read_ops(o0, sm, buf, 0, wm, wn, i32, g);
  read_ops(o1, sm, buf, 1, wm, wn, i32, g);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<FIRST>(o0, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  read_ops(o0, sm, buf, 2, wm, wn, i32, g);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o1, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  read_ops(o1, sm, buf, 3, wm, wn, i32, g);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o0, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
  mma_ops<false>(o1, Dlo, Dhi);
  __builtin_amdgcn_sched_barrier(0);
}

struct Ctx {
  int wm, wn, i32, g, lane;
};

/* acc += dA * (d * (Dlo + 8 Dhi) - dmin * sum_j m_j bsum_j) for one super-block */
__device__ __forceinline__ void epilogue(const Smem &sm, const Ctx &c, const v16i (&Dlo)[2],
                                         const v16i (&Dhi)[2], float (&acc)[2][16]) {
  const v16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const uint4 hd = sm.colhd[c.wn * 32 + c.i32];
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
    const v8h amin = *(const v8h *)(sm.amin + (rbase + c.i32) * 16 + c.g * 8);
    const v16f Sm = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const float4 dv = *(const float4 *)(sm.dA + rbase + 8 * q4 + 4 * c.g);
      const float dA[4] = {dv.x, dv.y, dv.z, dv.w};
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

/* One super-block. On entry LDS holds stage (sb, 0), the row/column data of sb,
 * and registers hold the weights of sb (bcur) and sb+1 (bnext). The order of the
 * global loads matters: the counters retire loads in issue order, so the far
 * prefetch of the weights (from HBM) is issued after the activation loads (L2
 * hits) that are needed first. */
__device__ __forceinline__ void super_block(Smem &sm, const Addr &ad, const Ctx &c, int sb,
                                            int nsb, BBlock &bcur, const BBlock &bnext,
                                            v16i (&Dlo)[2], v16i (&Dhi)[2],
                                            float (&acc)[2][16]) {
  AStage as;
  RowBlock rb;
  const int sb1 = min(sb + 1, nsb - 1), sb2 = min(sb + 2, nsb - 1);
  load_a(as, ad, sb, 1);
  __builtin_amdgcn_sched_barrier(0);
  stage_mma<true>(sm, 0, c.wm, c.wn, c.i32, c.g, Dlo, Dhi);
  store_a(as, sm, 1);
  store_b<1>(bcur, sm);
  sync_lds();
  load_a(as, ad, sb1, 0);
  load_row(rb, ad, sb1);
  load_b(bcur, ad, sb2); /* bcur's registers are free: they become the weights of sb + 2 */
  __builtin_amdgcn_sched_barrier(0);
  stage_mma<false>(sm, 1, c.wm, c.wn, c.i32, c.g, Dlo, Dhi);
  epilogue(sm, c, Dlo, Dhi, acc);
  sync_lds(); /* every wavefront is done with stage (sb, 0) and the row/column data */
  __builtin_amdgcn_sched_barrier(0);
  store_a(as, sm, 0);
  store_b<0>(bnext, sm);
  store_row(rb, sm);
  sync_lds();
}

__global__ __launch_bounds__(NT, 2) void gemm_q4k_kernel(WView w, QView qa, int M, int mtiles,
                                                         int ntiles, float *__restrict__ C,
                                                         int64_t ldc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem &sm = *reinterpret_cast<Smem *>(smem_raw);
  /* workgroup id -> tile: the M-tiles of one weight tile share id % 8 (one XCD) */
  const int id = blockIdx.x;
  const int xcd = id & 7, qd = id >> 3;
  const int mt = qd % mtiles, nt = (qd / mtiles) * 8 + xcd;
  if (nt >= ntiles) return; /* uniform per workgroup */
  const int m0 = mt * BM, n0 = nt * BN;
  Ctx c;
  c.lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  c.wm = wave >> 1;
  c.wn = wave & 1;
  c.i32 = c.lane & 31;
  c.g = c.lane >> 5;
  const int nsb = w.K >> 8;

  v16i Dlo[2], Dhi[2];
  float acc[2][16];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[a][r] = 0.f;

  const Addr ad = make_addr(w, qa, M, m0, n0);
  BBlock b0, b1;
  {
    AStage as;
    RowBlock rb;
    load_a(as, ad, 0, 0);
    load_row(rb, ad, 0);
    load_b(b0, ad, 0);
    load_b(b1, ad, min(1, nsb - 1));
    store_a(as, sm, 0);
    store_b<0>(b0, sm);
    store_row(rb, sm);
    sync_lds();
  }
  int sb = 0;
  for (; sb + 1 < nsb; sb += 2) {
    super_block(sm, ad, c, sb, nsb, b0, b1, Dlo, Dhi, acc);
    super_block(sm, ad, c, sb + 1, nsb, b1, b0, Dlo, Dhi, acc);
  }
  if (sb < nsb) super_block(sm, ad, c, sb, nsb, b0, b1, Dlo, Dhi, acc);

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

int launch_gemm_q4k(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc,
                    hipStream_t s) {
  const int mtiles = (M + BM - 1) / BM;
  const int ntiles = (int)((w->N + BN - 1) / BN);
  const int ngroups = (ntiles + 7) / 8;
  const unsigned grid = (unsigned)(mtiles * ngroups * 8);
  static bool lds_opt_in = false;
  if (!lds_opt_in) {
    HIPQ_HIP(hipFuncSetAttribute((const void *)gemm_q4k_kernel,
                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem)));
    lds_opt_in = true;
  }
  hipLaunchKernelGGL(gemm_q4k_kernel, dim3(grid), dim3(NT), sizeof(Smem), s, wview(w), qview(*qa),
                     M, mtiles, ntiles, C, ldc);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
