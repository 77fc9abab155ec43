// SPDX-License-Identifier: Apache-2.0
/**
 * @file   gemm.hip
 * @brief  Prefill GEMM (M > 8) for Q4_0 x Q8_0 on gfx950 int8 matrix cores.
 *         (Q4_K x Q8_K has its own kernel, gemm_q4k.hip.)
 *
 * Replaces the M > 1 branch of __ggml_q4_0_8x8_q8_0_GEMM
 * (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:330-389 in
 * the reference checkout) and the nntr_gemm_q4_0_8x8_q8_0 kernel behind it
 * (nntr_ggml_impl/nntr_ggml_impl.cpp:650-3259).
 *
 * What bounds it. Q4_0 has one fp16 scale per 32 weights and Q8_0 one per 32
 * activations, so a matrix instruction can cover one 32-deep block and no more, and
 * each of its exact int32 sums is scaled on the vector ALU:
 * acc += float(dot) * (dw * da), three instructions per sum per block, added in the
 * reference's block order (one fused multiply-add each), so the outputs carry the
 * reference's bits. That is 3 vector instructions per 32 multiply-adds: the vector
 * ALU, not the matrix core, sets the pace, and the vector ALU of a SIMD is only
 * busy when at least two wavefronts feed it (one wavefront issues a vector
 * instruction every 4.9 cycles, two together one every 2.45; measured).
 *
 * Structure. So the unit of work is small: a wavefront owns a 16 x 16 tile of C
 * (v_mfma_i32_16x16x32_i8, four sums a lane), a workgroup of 8 wavefronts a
 * 64 x 32 tile, and 512 rows by 1024 columns already make 256 workgroups, two
 * wavefronts on every SIMD of the chip. K is walked in chunks of 256. A chunk is
 * staged into one of two LDS buffers while the other is computed on (one barrier
 * per chunk), the global loads run two chunks ahead in two register sets, and the
 * LDS reads half a chunk ahead of the arithmetic that uses them. With two
 * wavefronts a SIMD a step of one chunk takes about 2250 cycles, 520 of them the
 * arithmetic of a wavefront: the rest is what two wavefronts cannot hide from each
 * other - the issue of the four vector-memory loads a wavefront makes per step
 * (about 200 cycles), 84 KB of LDS reads and 27 KB of LDS writes a workgroup and
 * step, and the wait of the early wavefronts at the barrier. Grids with more than
 * one workgroup per CU (wide N) hide more of it.
 * Per chunk a workgroup stages
 *   - the int8 activations of its 64 rows (16 KB),
 *   - the int8 expansion of its 32 weight rows: nibbles are unpacked in registers
 *     on the way from HBM to LDS, so HBM only ever carries the packed 4.5-bit form,
 *   - the scales of both sides as fp32.
 * The bytes of a row are stored in the order the matrix instruction wants them:
 * lane (i, g) of v_mfma_i32_16x16x32_i8 takes bytes 8 g .. 8 g + 7 of a block, so a
 * row is laid out [g][block][8 bytes] and a lane fetches its share of two blocks
 * with one 128-bit read (rows padded to 272 bytes: the 16 lanes of a read phase hit
 * 16 disjoint 4-bank groups). In the result layout a lane holds one column n and
 * 4 consecutive rows m: the weight scales of a chunk are two 128-bit reads
 * ([column][block]); the activation scales ([block][row]) are spread over the 16
 * lanes of a DPP row and broadcast inside the multiply that uses them.
 */
#include "gemv_device.h"

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int BM = 64, BN = 32, KC = 256, NT = 512;
constexpr int LDS_STRIDE = KC + 16; /* bytes per staged row */

struct SmemQ40 { /* one of the two chunk buffers */
  int8_t a[BM * LDS_STRIDE]; /* row: [g 0..3][block 0..7][8 bytes] */
  int8_t b[BN * LDS_STRIDE];
  float da[8 * BM]; /* [block in chunk][row] */
  float dw[BN * 8]; /* [column][block in chunk] */
};
static_assert(sizeof(SmemQ40) * 2 * 2 <= 160 * 1024, "two workgroups per CU, two buffers each");

/* A weight q - 8 enters the matrix instruction as 16 (q - 8): with bit 3 of every nibble flipped the
 * nibble IS q - 8 in two's complement, and in the high half of a byte that is the int8 value
 * 16 (q - 8) - one exclusive-or for eight weights, then a mask for the odd and a shift and a mask
 * for the even ones (how the reference reads its repacked blocks, nntr_ggml_impl.cpp:3233-3240). The
 * sums are 16 times too large, exactly (|16 dot| < 2^20), and the weight scales are staged as dw / 16
 * (a power of two: fl((dw / 16) da) = fl(dw da) / 16 for every fp16 pair of scales), so
 * fma(float(16 dot), fl(dw da) / 16, acc) has the operands' exact product of the reference's
 * fma(float(dot), fl(dw da), acc) and rounds to the same bits. */
constexpr uint32_t HIPQ_MHI = 0xf0f0f0f0u;

/* One chunk of a workgroup's inputs, as loaded (registers of one thread). Every thread takes the
 * same share of the staging, so that no wavefront keeps the others waiting at the barrier. */
struct Chunk {
  v4i a[2]; /* activations: piece idx = it * 512 + t -> row idx / 16, 16-byte column idx % 16 */
  uint2 x;  /* nibbles: half t & 1 (dwords 0, 1 or 2, 3) of block (t / 2) % 8 of column t / 16 */
  uint4 sc; /* t < 32: the 8 fp16 weight scales of column t. 32 <= t < 160: 4 of the 8 metadata
               words (fp16 d in the low half) of row (t - 32) / 2, blocks 4 * (t & 1) .. + 3.
               Wavefronts above that load none. */
};

/* Where a thread's loads of chunk 0 start, as byte offsets from the workgroup's first row and
 * first column (they fit 32 bits: at most 64 rows of K bytes), computed once. */
struct LoadOffsets {
  uint32_t a[2], x, sc;
  bool sc_is_dw;
};

__device__ __forceinline__ LoadOffsets load_offsets(const WView &w, const QView &qa, int M, int m0, int n0) {
  const int t = threadIdx.x;
  const int nb = w.K >> 5;
  LoadOffsets o;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * NT + t;
    const int row = min(idx >> 4, M - 1 - m0); /* rows past M repeat the last; they are never stored */
    o.a[it] = (uint32_t)row * (uint32_t)qa.K + (idx & 15) * 16;
  }
  const int col = min(t >> 4, w.N - 1 - n0);
  o.x = (uint32_t)col * (uint32_t)(w.K >> 1) + ((t >> 1) & 7) * 16 + (t & 1) * 8;
  o.sc_is_dw = t < 32;
  const int scol = min(t & 31, w.N - 1 - n0);
  const int srow = min(((t - 32) >> 1) & 63, M - 1 - m0);
  o.sc = o.sc_is_dw ? (uint32_t)scol * nb * 2 : (uint32_t)srow * nb * 4 + 16 * (t & 1);
  return o;
}

/* Bases of the workgroup's tile (uniform). */
struct TileBases {
  const int8_t *a;
  const uint8_t *x;
  const uint8_t *dw, *ma;
};

__device__ __forceinline__ void load_chunk(Chunk &c, const TileBases &tb, const LoadOffsets &o, int kc) {
  const int8_t *pa = tb.a + (size_t)kc * KC; /* uniform: the loads take it from scalar registers */
  c.a[0] = *(const v4i *)(pa + o.a[0]);
  c.a[1] = *(const v4i *)(pa + o.a[1]);
  c.x = *(const uint2 *)(tb.x + (size_t)kc * (KC / 2) + o.x);
  if (threadIdx.x < 192) { /* three wavefronts; the third's upper half fetches spare copies */
    const uint8_t *ps = o.sc_is_dw ? tb.dw + (size_t)kc * 16 : tb.ma + (size_t)kc * 32;
    c.sc = *(const uint4 *)(ps + o.sc);
  }
}

__device__ __forceinline__ void store_chunk(const Chunk &c, SmemQ40 &sm) {
  const int t = threadIdx.x;
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int idx = it * NT + t;
    const int c16 = idx & 15; /* bytes 16 c16 .. + 15 of the row: block c16 / 2, g = 2 (c16 & 1), + 1 */
    int8_t *dst = sm.a + (idx >> 4) * LDS_STRIDE + (c16 & 1) * 128 + (c16 >> 1) * 8;
    *(v2i *)dst = v2i{c.a[it][0], c.a[it][1]};
    *(v2i *)(dst + 64) = v2i{c.a[it][2], c.a[it][3]};
  }
  {
    /* a 32-value block is 16 bytes: low nibbles = elements 0..15, high = 16..31. Dwords 0, 1 carry
     * elements 0..7 (g = 0) and 16..23 (g = 2), dwords 2, 3 elements 8..15 (g = 1) and 24..31 (g = 3). */
    const int h = t & 1;
    int8_t *dst = sm.b + (t >> 4) * LDS_STRIDE + h * 64 + ((t >> 1) & 7) * 8;
    const uint32_t x0 = c.x.x ^ 0x88888888u, x1 = c.x.y ^ 0x88888888u;
    *(v2i *)dst = v2i{(int)((x0 << 4) & HIPQ_MHI), (int)((x1 << 4) & HIPQ_MHI)};
    *(v2i *)(dst + 128) = v2i{(int)(x0 & HIPQ_MHI), (int)(x1 & HIPQ_MHI)};
  }
  const uint32_t s4[4] = {c.sc.x, c.sc.y, c.sc.z, c.sc.w};
  if (t < 32) {
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = hipq_h2f((uint16_t)(s4[i] & 0xffff)) * 0.0625f; /* exact: see above */
      f[2 * i + 1] = hipq_h2f((uint16_t)(s4[i] >> 16)) * 0.0625f;
    }
    float4 *dst = (float4 *)(sm.dw + t * 8);
    dst[0] = float4{f[0], f[1], f[2], f[3]};
    dst[1] = float4{f[4], f[5], f[6], f[7]};
  } else if (t < 160) {
    const int row = (t - 32) >> 1, b0 = 4 * (t & 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) sm.da[(b0 + i) * BM + row] = hipq_h2f((uint16_t)(s4[i] & 0xffff));
  }
}

/* da * dw with da taken from lane R of the DPP row (16 lanes) inside the multiply itself */
#define HIPQ_MUL_BCAST(DA, DW, R)                                                                   \
  ({                                                                                                \
    float t_;                                                                                       \
    asm("v_mul_f32_dpp %0, %1, %2 row_newbcast:" #R " row_mask:0xf bank_mask:0xf"                   \
        : "=v"(t_)                                                                                  \
        : "v"(DA), "v"(DW));                                                                        \
    t_;                                                                                             \
  })

/* What one wavefront's 16 x 16 tile needs of four blocks (half a chunk): its lane's 8 bytes of
 * each block on both sides (av[p]: blocks 2 p and 2 p + 1) and the four weight scales of its column. */
struct Half {
  v4i av[2], bv[2];
  float4 dw;
};

struct LaneOffsets {
  int a, b, dw, da;
};

__device__ __forceinline__ void read_half(Half &hf, const SmemQ40 &sm, const LaneOffsets &o, int half) {
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    hf.av[p] = *(const v4i *)(sm.a + o.a + (2 * half + p) * 16);
    hf.bv[p] = *(const v4i *)(sm.b + o.b + (2 * half + p) * 16);
  }
  hf.dw = *(const float4 *)(sm.dw + o.dw + 4 * half);
}

/* The 32 activation scales a DPP row needs of a chunk (4 rows x 8 blocks) are spread two a lane
 * over the row's 16 lanes (one 64-bit read) and broadcast by the multiply that uses them: reading
 * them as 128-bit words a block would be 8 KB of LDS traffic a wavefront and chunk, as much as
 * both operands. */
__device__ __forceinline__ float2 read_da(const SmemQ40 &sm, const LaneOffsets &o) {
  return *(const float2 *)(sm.da + o.da);
}

__device__ __forceinline__ v4i block_dot(const Half &hf, int j) {
  const v4i zero4 = {0, 0, 0, 0};
  const int h = 2 * (j & 1);
  const long a8 = (long)(uint32_t)hf.av[j >> 1][h] | ((long)hf.av[j >> 1][h + 1] << 32);
  const long b8 = (long)(uint32_t)hf.bv[j >> 1][h] | ((long)hf.bv[j >> 1][h + 1] << 32);
  return __builtin_amdgcn_mfma_i32_16x16x32_i8(a8, b8, zero4, 0, 0, 0);
}

/* acc += float(dot) * (dw * da) on the four sums of a block; the activation scales of rows
 * 4 g + 0, 1 sit in lane R0 of the DPP row, those of rows 4 g + 2, 3 in lane R1 */
#define HIPQ_Q40_CHAIN(DOT, DW, R0, R1)                                                             \
  {                                                                                                 \
    acc[0] = fmaf((float)(DOT)[0], HIPQ_MUL_BCAST(dar.x, DW, R0), acc[0]);                          \
    acc[1] = fmaf((float)(DOT)[1], HIPQ_MUL_BCAST(dar.y, DW, R0), acc[1]);                          \
    acc[2] = fmaf((float)(DOT)[2], HIPQ_MUL_BCAST(dar.x, DW, R1), acc[2]);                          \
    acc[3] = fmaf((float)(DOT)[3], HIPQ_MUL_BCAST(dar.y, DW, R1), acc[3]);                          \
  }

__device__ __forceinline__ void pin(float (&acc)[4]) {
  /* pins the chains before it to this place in the instruction stream (the compiler otherwise
   * may sink them below the staging that follows and keep their operands alive across it) */
#pragma unroll
  for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(acc[r]));
}

/* Four blocks. The matrix instruction of block j + 1 is issued before the chain of block j, so
 * the chain never waits for its sums. */
__device__ __forceinline__ void compute_first_half(const Half &hf, float2 dar, float (&acc)[4]) {
  const v4i d0 = block_dot(hf, 0);
  const v4i d1 = block_dot(hf, 1);
  HIPQ_Q40_CHAIN(d0, hf.dw.x, 0, 1)
  const v4i d2 = block_dot(hf, 2);
  HIPQ_Q40_CHAIN(d1, hf.dw.y, 2, 3)
  const v4i d3 = block_dot(hf, 3);
  HIPQ_Q40_CHAIN(d2, hf.dw.z, 4, 5)
  HIPQ_Q40_CHAIN(d3, hf.dw.w, 6, 7)
  pin(acc);
}

__device__ __forceinline__ void compute_second_half(const Half &hf, float2 dar, float (&acc)[4]) {
  const v4i d0 = block_dot(hf, 0);
  const v4i d1 = block_dot(hf, 1);
  HIPQ_Q40_CHAIN(d0, hf.dw.x, 8, 9)
  const v4i d2 = block_dot(hf, 2);
  HIPQ_Q40_CHAIN(d1, hf.dw.y, 10, 11)
  const v4i d3 = block_dot(hf, 3);
  HIPQ_Q40_CHAIN(d2, hf.dw.z, 12, 13)
  HIPQ_Q40_CHAIN(d3, hf.dw.w, 14, 15)
  pin(acc);
}

/* Up to four weights of one K against the same activations as ONE launch: the grid's columns are
 * the concatenation of the weights' column tiles (Q, K, V or gate, up of a layer: three or two
 * small grids become one that fills the chip, and two launches fewer). */
struct MultiQ40 {
  WView w[4];
  float *C[4];
  int64_t ldc[4];
  int tile_end[4]; /* running sum of the weights' column tiles */
};

__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_q40_kernel(
  MultiQ40 mw, QView qa, int M) {
  __shared__ SmemQ40 smb[2];
  /* which weight this workgroup's column tile belongs to (uniform) */
  int bx = blockIdx.x, wi = 0;
  if (bx >= mw.tile_end[0]) wi = 1;
  if (bx >= mw.tile_end[1]) wi = 2;
  if (bx >= mw.tile_end[2]) wi = 3;
  if (wi) bx -= mw.tile_end[wi - 1];
  const WView w = wi == 0 ? mw.w[0] : wi == 1 ? mw.w[1] : wi == 2 ? mw.w[2] : mw.w[3];
  float *__restrict__ C = wi == 0 ? mw.C[0] : wi == 1 ? mw.C[1] : wi == 2 ? mw.C[2] : mw.C[3];
  const int64_t ldc = wi == 0 ? mw.ldc[0] : wi == 1 ? mw.ldc[1] : wi == 2 ? mw.ldc[2] : mw.ldc[3];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1; /* 4 x 2 wavefronts, 16 x 16 each */
  const int n0 = bx * BN, m0 = blockIdx.y * BM;
  const int i16 = lane & 15, g = lane >> 4;
  const int nchunks = w.K / KC;
  const int nb = w.K >> 5;
  /* the lane's sums are rows 4 g .. 4 g + 3, column i16; lane i16 of a DPP row keeps the
   * activation scales of block i16 / 2, rows 4 g + 2 (i16 & 1) and the next */
  LaneOffsets o;
  o.a = (wm * 16 + i16) * LDS_STRIDE + g * 64;
  o.b = (wn * 16 + i16) * LDS_STRIDE + g * 64;
  o.dw = (wn * 16 + i16) * 8;
  o.da = (i16 >> 1) * BM + wm * 16 + 4 * g + 2 * (i16 & 1);
  const LoadOffsets lo = load_offsets(w, qa, M, m0, n0);
  TileBases tb;
  tb.a = qa.q + (size_t)m0 * qa.K;
  tb.x = w.qs + (size_t)n0 * (w.K >> 1);
  tb.dw = (const uint8_t *)(w.d + (size_t)n0 * nb);
  tb.ma = (const uint8_t *)(qa.meta + (size_t)m0 * nb);

  float acc[4] = {0.f, 0.f, 0.f, 0.f};

  /* Global to LDS: two register sets hold the chunks one and two steps ahead of the one in LDS
   * last; a set is written to LDS two steps after its loads were issued and then takes the loads
   * of the chunk after next.
   * LDS to registers: the operands travel half a chunk ahead of their use. A step starts, right
   * after the barrier that published chunk c, by requesting chunk c's first half; then it stages
   * chunk c + 1 into the buffer chunk c - 1 was in (whose reads all finished before that barrier),
   * issues the global loads of chunk c + 3, computes the second half of chunk c - 1, requests
   * chunk c's second half and computes its first half. Every LDS read and write so has the
   * length of a half chunk's arithmetic to complete before something waits for it. */
  Chunk r0, r1;
  Half h0, h1;
  float2 dar, dar_next;
  const int last = nchunks - 1; /* loads past the end repeat the last chunk; what they store is not read */
  load_chunk(r0, tb, lo, 0);
  load_chunk(r1, tb, lo, min(1, last));
  store_chunk(r0, smb[0]);
  load_chunk(r0, tb, lo, min(2, last));
  __syncthreads();
  read_half(h0, smb[0], o, 0);
  dar = read_da(smb[0], o);
  read_half(h1, smb[0], o, 1);
  compute_first_half(h0, dar, acc);
  store_chunk(r1, smb[1]);
  load_chunk(r1, tb, lo, min(3, last));
  __syncthreads();
  for (int c = 1; c < nchunks; c += 2) {
    /* odd step: chunk c is in buffer 1, r0 holds chunk c + 1 */
    read_half(h0, smb[1], o, 0);
    dar_next = read_da(smb[1], o);
    store_chunk(r0, smb[0]);
    load_chunk(r0, tb, lo, min(c + 3, last));
    compute_second_half(h1, dar, acc);
    read_half(h1, smb[1], o, 1);
    dar = dar_next;
    compute_first_half(h0, dar, acc);
    __syncthreads();
    if (c + 1 >= nchunks) break;
    /* even step: chunk c + 1 is in buffer 0, r1 holds chunk c + 2 */
    read_half(h0, smb[0], o, 0);
    dar_next = read_da(smb[0], o);
    store_chunk(r1, smb[1]);
    load_chunk(r1, tb, lo, min(c + 4, last));
    compute_second_half(h1, dar, acc);
    read_half(h1, smb[0], o, 1);
    dar = dar_next;
    compute_first_half(h0, dar, acc);
    __syncthreads();
  }
  compute_second_half(h1, dar, acc);

  const int n = n0 + wn * 16 + i16;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = m0 + wm * 16 + 4 * g + r;
    if (m < M && n < w.N) C[(int64_t)m * ldc + n] = acc[r];
  }
}

} // namespace

namespace hipq {

static int check_gemm_weight(const hipq_weight *w) {
  if (w->K % KC) return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm needs K %% 256 == 0, got %lld", (long long)w->K);
  if (w->dtype != HIPQ_Q4_0) return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm: dtype %d has no MFMA path here", w->dtype);
  if ((int64_t)BM * w->K >= (int64_t)1 << 31)
    return fail(HIPQ_ERR_NOT_SUPPORTED, "gemm: K = %lld is beyond the kernel's 32-bit tile offsets", (long long)w->K);
  return HIPQ_OK;
}

int launch_gemm_multi(int count, const hipq_weight *const *w, const QAct *qa, int M, float *const *C,
                      const int64_t *ldc, hipStream_t s) {
  if (count < 1 || count > 4) return fail(HIPQ_ERR_INVALID_ARGUMENT, "gemm: 1 to 4 weights per launch, got %d", count);
  MultiQ40 mw;
  int tiles = 0;
  for (int i = 0; i < 4; ++i) {
    const hipq_weight *wi = w[i < count ? i : count - 1];
    if (i < count) {
      if (int rc = check_gemm_weight(wi)) return rc;
      if (wi->K != w[0]->K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "gemm: the weights of one launch share K");
      tiles += (int)((wi->N + BN - 1) / BN);
    }
    mw.w[i] = wview(wi);
    mw.C[i] = C[i < count ? i : count - 1];
    mw.ldc[i] = ldc[i < count ? i : count - 1];
    mw.tile_end[i] = tiles; /* unused entries repeat the total: no workgroup lands in them */
  }
  const dim3 grid((unsigned)tiles, (unsigned)((M + BM - 1) / BM));
  hipq::launch_kernel("gemm_q40_kernel", gemm_q40_kernel, grid, dim3(NT), 0, s, mw, qview(*qa), M);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

int launch_gemm(const hipq_weight *w, const QAct *qa, int M, float *C, int64_t ldc,
                hipStream_t s) {
  return launch_gemm_multi(1, &w, qa, M, &C, &ldc, s);
}

} // namespace hipq
