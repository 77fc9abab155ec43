// SPDX-License-Identifier: Apache-2.0
/**
 * @file   relayout.hip
 * @brief  One-time conversion of ggml weight blocks (canonical rows, or the
 *         8-row interleave NNTrainer stores on disk) into the plane layout the
 *         gfx950 kernels read (see hipq_internal.h).
 *
 * Inverse of the reference's repack (nntr_make_block_q4_0x8 /
 * make_block_q4_Kx8, nntrainer/tensor/cpu_backend/ggml_interface/
 * nntr_ggml_impl/nntr_ggml_impl.cpp:8056-8158 in the reference checkout) fused
 * with the array-of-structs -> planes split. Pure byte movement; runs once per
 * weight at load time, one thread per source block.
 */
#include <mutex>

#include "hipq_internal.h"

namespace {

/* 6-bit scale/min j of a 12-byte packed group (get_scale_min_k4). */
__device__ __forceinline__ void scale_min(int j, const uint8_t *s, int &sc, int &mn) {
  if (j < 4) {
    sc = s[j] & 63;
    mn = s[j + 4] & 63;
  } else {
    sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
    mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
  }
}

__global__ void relayout_q4_0(const uint8_t *__restrict__ src, int x8, int64_t N, int nb,
                              uint8_t *__restrict__ qs, uint16_t *__restrict__ d) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * nb) return;
  const int64_t n = i / nb;
  const int b = (int)(i - n * nb);
  uint8_t *oq = qs + i * 16;
  if (!x8) {
    const uint8_t *blk = src + i * 18;
    d[i] = (uint16_t)(blk[0] | (blk[1] << 8));
    for (int k = 0; k < 16; ++k) oq[k] = blk[2 + k];
  } else {
    const int r = (int)(n & 7);
    const uint8_t *grp = src + ((n >> 3) * nb + b) * 144;
    d[i] = (uint16_t)(grp[2 * r] | (grp[2 * r + 1] << 8));
    for (int k = 0; k < 16; ++k)
      oq[k] = grp[16 + (k >> 3) * 64 + r * 8 + (k & 7)] ^ 0x88;
  }
}

__global__ void relayout_q4_K(const uint8_t *__restrict__ src, int x8, int64_t N, int nb,
                              uint8_t *__restrict__ qs, uint8_t *__restrict__ hdr) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * nb) return;
  const int64_t n = i / nb;
  const int b = (int)(i - n * nb);
  uint8_t *oq = qs + i * 128;
  uint8_t *oh = hdr + i * 16;
  uint8_t sc[8], mn[8]; /* the super-block's 6-bit scales and mins */
  uint8_t cq[128]; /* the super-block's qs in the byte order of block_q4_K */
  if (!x8) {
    const uint8_t *blk = src + i * 144;
    for (int k = 0; k < 4; ++k) oh[k] = blk[k];
    const uint8_t *s = blk + 4; /* the 12 packed bytes of block_q4_K */
    for (int j = 0; j < 4; ++j) {
      sc[j] = s[j] & 63;
      mn[j] = s[j + 4] & 63;
      sc[j + 4] = (uint8_t)((s[j + 8] & 0x0f) | ((s[j] >> 6) << 4));
      mn[j + 4] = (uint8_t)((s[j + 8] >> 4) | ((s[j + 4] >> 6) << 4));
    }
    for (int k = 0; k < 128; ++k) cq[k] = blk[16 + k];
  } else {
    const int r = (int)(n & 7);
    const uint8_t *grp = src + ((n >> 3) * nb + b) * 1152;
    oh[0] = grp[2 * r];
    oh[1] = grp[2 * r + 1];
    oh[2] = grp[16 + 2 * r];
    oh[3] = grp[16 + 2 * r + 1];
    /* group g of the interleaved scales holds sub-block g of all 8 rows,
     * indexed by row */
    for (int g = 0; g < 8; ++g) {
      int s1, m1;
      scale_min(r, grp + 32 + 12 * g, s1, m1);
      sc[g] = (uint8_t)s1;
      mn[g] = (uint8_t)m1;
    }
    for (int k = 0; k < 128; ++k) cq[k] = grp[128 + (k >> 3) * 64 + r * 8 + (k & 7)];
  }
  /* each sub-block's scale in a byte of its own with the top two bits of its min
   * above it, then the low four bits of the mins of sub-blocks k and k + 4 per byte */
  for (int j = 0; j < 8; ++j) oh[4 + j] = (uint8_t)(sc[j] | ((mn[j] >> 4) << 6));
  for (int k = 0; k < 4; ++k) oh[12 + k] = (uint8_t)((mn[k] & 15) | ((mn[k + 4] & 15) << 4));
  /* block_q4_K keeps sub-blocks 2c / 2c+1 in the low / high nibbles of 32 bytes.
   * The device plane stores each sub-block's 32 weights as 16 consecutive bytes,
   * weight 2i in the low and 2i+1 in the high nibble of byte i, so that one
   * dword is eight weights of ONE sub-block (the unit of v_dot8_u32_u4). */
  for (int j = 0; j < 8; ++j) {
    const uint8_t *ch = cq + 32 * (j >> 1);
    const int sh = 4 * (j & 1);
    for (int k = 0; k < 16; ++k)
      oq[16 * j + k] = (uint8_t)(((ch[2 * k] >> sh) & 15) | (((ch[2 * k + 1] >> sh) & 15) << 4));
  }
}

__global__ void relayout_q6_K(const uint8_t *__restrict__ src, int64_t total,
                              uint8_t *__restrict__ ql, uint8_t *__restrict__ qh,
                              int8_t *__restrict__ sc, uint16_t *__restrict__ d) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const uint8_t *blk = src + i * 210;
  /* ql in two planes: unit uu = half * 2 + hl takes bytes half*64 + hl*16 .. +15 (low
   * nibbles: elements l, high: l + 64) from the first and the 16 bytes 32 further on
   * (elements l + 32, l + 96) from the second, so that the units of a row are
   * consecutive 16-byte pieces in both */
  uint8_t *qlb = ql + total * 64;
  for (int uu = 0; uu < 4; ++uu)
    for (int t = 0; t < 16; ++t) {
      const int o = (uu >> 1) * 64 + (uu & 1) * 16 + t;
      ql[i * 64 + uu * 16 + t] = blk[o];
      qlb[i * 64 + uu * 16 + t] = blk[o + 32];
    }
  for (int k = 0; k < 64; ++k) qh[i * 64 + k] = blk[128 + k];
  for (int u = 0; u < 4; ++u)
    for (int g = 0; g < 4; ++g)
      sc[i * 16 + u * 4 + g] = (int8_t)blk[192 + (u >> 1) * 8 + g * 2 + (u & 1)];
  d[i] = (uint16_t)(blk[208] | (blk[209] << 8));
}

/* planes -> tiles of 32 rows for the expert kernels (4096 bytes of nibbles, then the 512 bytes of
 * headers, per tile and super-block): thread = one 16-byte piece of nibbles */
__global__ void tile_q4_K(const uint8_t *__restrict__ qs, const uint8_t *__restrict__ hdr, int N, int nsb,
                          int64_t pieces, uint8_t *__restrict__ tq) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= pieces) return;
  const int lane = (int)(p & 63), i = (int)((p >> 6) & 3);
  const int64_t ts = p >> 8; /* tile * nsb + sb */
  const int sb = (int)(ts % nsb);
  const int64_t tile = ts / nsb;
  const int64_t n = tile * 32 + (lane & 31);
  const int g = lane >> 5;
  uint2 a = make_uint2(0, 0), b = make_uint2(0, 0);
  if (n < N) {
    const uint8_t *src = qs + (n * nsb + sb) * 128 + g * 8;
    a = *(const uint2 *)(src + (2 * i) * 16);
    b = *(const uint2 *)(src + (2 * i + 1) * 16);
  }
  uint8_t *dst = tq + ts * hipq::EXPERT_TILE_BYTES;
  *(uint4 *)(dst + (p & 255) * 16) = make_uint4(a.x, a.y, b.x, b.y);
  if (i == 0 && g == 0)
    *(uint4 *)(dst + 4096 + (lane & 31) * 16) =
      n < N ? *(const uint4 *)(hdr + (n * nsb + sb) * 16) : make_uint4(0, 0, 0, 0);
}

/* planes -> tiles of 32 rows for the prefill GEMM: thread = one 16-byte piece,
 * piece (i, lane (n, g)) = sub-block 4g + i of row n */
__global__ void gemm_tile_q4_K(const uint8_t *__restrict__ qs, const uint8_t *__restrict__ hdr, int N, int nsb,
                               int64_t pieces, uint8_t *__restrict__ tq, uint8_t *__restrict__ th) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= pieces) return;
  const int lane = (int)(p & 63), i = (int)((p >> 6) & 3);
  const int64_t ts = p >> 8; /* tile * nsb + sb */
  const int sb = (int)(ts % nsb);
  const int64_t n = (ts / nsb) * 32 + (lane & 31);
  const int g = lane >> 5;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (n < N) v = *(const uint4 *)(qs + (n * nsb + sb) * 128 + (4 * g + i) * 16);
  *(uint4 *)(tq + p * 16) = v;
  if (i == 0 && g == 0)
    *(uint4 *)(th + (ts * 32 + (lane & 31)) * 16) =
      n < N ? *(const uint4 *)(hdr + (n * nsb + sb) * 16) : make_uint4(0, 0, 0, 0);
}

/* Q6_K planes -> tiles of 32 rows for the prefill GEMM (hipq_internal.h, gt_qs / gt_qh / gt_hdr
 * of a Q6_K weight): thread = lane (n, g) of one (tile, super-block), which owns half g of
 * row n's super-block. In block_q6_K order the half's 128 weights are four quarters of 32:
 * quarter c takes its low four bits from the low (c < 2) or high nibbles of ql bytes
 * 64 g + 32 (c & 1) .. + 31 and its bits 4-5 from bits 2c, 2c+1 of qh bytes 32 g .. + 31
 * (dequantize_row_q6_K, nntr_ggml_impl_quant.cpp:1291-1325). Step s of the lane = weights
 * 16 s .. 16 s + 15 of the half = bytes 16 (s & 1) .. + 15 of quarter s >> 1. The planes
 * hold ql bytes 64 g + 16 u + t (u = 0, 1) at unit 2g + u of the first plane and the bytes
 * 32 further on at the same place of the second (relayout_q6_K above). */
__global__ void gemm_tile_q6_K(const uint8_t *__restrict__ ql, const uint8_t *__restrict__ qh,
                               const int8_t *__restrict__ sc, const uint16_t *__restrict__ d, int N, int nsb,
                               int64_t total_sb, int64_t lanes, uint8_t *__restrict__ tq, uint8_t *__restrict__ th,
                               uint8_t *__restrict__ thd) {
  const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= lanes) return;
  const int lane = (int)(p & 63);
  const int64_t ts = p >> 6; /* tile * nsb + sb */
  const int sb = (int)(ts % nsb);
  const int64_t n = (ts / nsb) * 32 + (lane & 31);
  const int g = lane >> 5;
  uint32_t x[8][2], hb[8];
  uint32_t hdr[4] = {0, 0, 0, 0};
  for (int s = 0; s < 8; ++s) x[s][0] = x[s][1] = hb[s] = 0;
  if (n < N) {
    const int64_t i = n * nsb + sb;
    const uint8_t *qlb = ql + total_sb * 64;
    for (int s = 0; s < 8; ++s) {
      const int c = s >> 1;
      const uint8_t *nib = ((c & 1) ? qlb : ql) + i * 64 + (2 * g + (s & 1)) * 16;
      const uint8_t *hi = qh + i * 64 + 32 * g + 16 * (s & 1);
      uint32_t w4[16], w2[16];
      for (int k = 0; k < 16; ++k) {
        w4[k] = (c < 2) ? (nib[k] & 15u) : (uint32_t)(nib[k] >> 4);
        w2[k] = (hi[k] >> (2 * c)) & 3u;
      }
      for (int k = 0; k < 4; ++k) {
        x[s][0] |= (w4[2 * k] | (w4[2 * k + 1] << 4)) << (8 * k);
        x[s][1] |= (w4[8 + 2 * k] | (w4[8 + 2 * k + 1] << 4)) << (8 * k);
        hb[s] |= (w2[2 * k] | (w2[2 * k + 8] << 2) | (w2[2 * k + 1] << 4) | (w2[2 * k + 9] << 6)) << (8 * k);
      }
      /* the scale of weights 128 g + 16 s .. + 15 is scales[8 g + s]; the plane keeps scale j of
       * half h at (2 h + (j & 1)) * 4 + ((j & 7) >> 1) */
      const uint32_t sv = (uint8_t)sc[i * 16 + (2 * g + (s & 1)) * 4 + (s >> 1)];
      hdr[s >> 2] |= sv << (8 * (s & 3));
    }
    hdr[2] = d[i];
  }
  for (int q = 0; q < 4; ++q)
    *(uint4 *)(tq + ((ts * 4 + q) * 64 + lane) * 16) = make_uint4(x[2 * q][0], x[2 * q][1], x[2 * q + 1][0], x[2 * q + 1][1]);
  for (int q = 0; q < 2; ++q)
    *(uint4 *)(th + ((ts * 2 + q) * 64 + lane) * 16) = make_uint4(hb[4 * q], hb[4 * q + 1], hb[4 * q + 2], hb[4 * q + 3]);
  *(uint4 *)(thd + (ts * 64 + lane) * 16) = make_uint4(hdr[0], hdr[1], hdr[2], hdr[3]);
}

} // namespace

namespace hipq {

int ensure_gemm_tiles(hipq_weight *w) {
  static std::mutex mu; /* two threads may run their first prefill product on one weight */
  std::lock_guard<std::mutex> lk(mu);
  if (w->gt_base) return HIPQ_OK;
  if ((w->dtype != HIPQ_Q4_K && w->dtype != HIPQ_Q6_K) || w->expert_tiles)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "only Q4_K and Q6_K weights in the plane layout have a GEMM tile copy");
  const int nsb = (int)(w->K / 256);
  const int64_t tiles = (w->N + 31) / 32;
  const bool q6 = w->dtype == HIPQ_Q6_K;
  /* Q4_K: nibbles, headers. Q6_K: nibbles, high bits, scales (every part a multiple of 256 bytes) */
  const size_t q_bytes = (size_t)tiles * nsb * 4096, x_bytes = q6 ? (size_t)tiles * nsb * 2048 : 0,
               h_bytes = (size_t)tiles * nsb * (q6 ? 1024 : 512);
  uint8_t *nb = nullptr;
  hipError_t e = hipMalloc((void **)&nb, q_bytes + x_bytes + h_bytes);
  if (e != hipSuccess)
    return fail(HIPQ_ERR_OUT_OF_MEMORY, "GEMM tiles of %zu bytes: %s", q_bytes + x_bytes + h_bytes, hipGetErrorString(e));
  if (q6) {
    const int64_t lanes = tiles * nsb * 64;
    hipq::launch_kernel("gemm_tile_q6_K", gemm_tile_q6_K, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, nullptr, w->qs, w->qh, w->sc,
                       w->d, (int)w->N, nsb, (int64_t)w->N * nsb, lanes, nb, nb + q_bytes, nb + q_bytes + x_bytes);
  } else {
    const int64_t pieces = tiles * nsb * 256;
    hipq::launch_kernel("gemm_tile_q4_K", gemm_tile_q4_K, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, nullptr, w->qs, w->hdr,
                       (int)w->N, nsb, pieces, nb, nb + q_bytes);
  }
  e = hipGetLastError();
  if (e == hipSuccess) e = hipStreamSynchronize(nullptr); /* the caller's stream may be another one */
  if (e != hipSuccess) {
    (void)hipFree(nb);
    return fail(HIPQ_ERR_RUNTIME, "GEMM tiling: %s", hipGetErrorString(e));
  }
  w->gt_qs = nb;
  w->gt_qh = q6 ? nb + q_bytes : nullptr;
  w->gt_hdr = nb + q_bytes + x_bytes;
  w->gt_base = nb; /* last: readers test this field */
  return HIPQ_OK;
}

int tile_expert_weight(hipq_weight *w) {
  if (w->dtype != HIPQ_Q4_K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "only Q4_K weights have an expert layout");
  if (w->expert_tiles) return HIPQ_OK;
  const int nsb = (int)(w->K / 256);
  const int64_t tiles = (w->N + 31) / 32;
  const size_t bytes = (size_t)tiles * nsb * EXPERT_TILE_BYTES;
  uint8_t *nb = nullptr;
  hipError_t e = hipMalloc((void **)&nb, bytes);
  if (e != hipSuccess) return fail(HIPQ_ERR_OUT_OF_MEMORY, "expert tiles of %zu bytes: %s", bytes, hipGetErrorString(e));
  const int64_t pieces = tiles * nsb * 256;
  hipq::launch_kernel("tile_q4_K", tile_q4_K, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, nullptr, w->qs, w->hdr,
                     (int)w->N, nsb, pieces, nb);
  e = hipGetLastError();
  if (e == hipSuccess) e = hipDeviceSynchronize(); /* nothing may still read the planes that are freed next */
  if (e != hipSuccess) {
    (void)hipFree(nb);
    return fail(HIPQ_ERR_RUNTIME, "expert tiling: %s", hipGetErrorString(e));
  }
  (void)hipFree(w->base);
  w->base = nb;
  w->bytes = bytes;
  w->qs = nb;
  w->hdr = nb + 4096;
  w->expert_tiles = 1;
  return HIPQ_OK;
}

int launch_relayout(hipq_weight *w, int layout, const uint8_t *src, hipStream_t s) {
  const int x8 = layout == HIPQ_LAYOUT_X8;
  if (w->dtype == HIPQ_Q4_0) {
    const int nb = (int)(w->K / 32);
    const int64_t total = w->N * nb;
    hipq::launch_kernel("relayout_q4_0", relayout_q4_0, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, src,
                       x8, w->N, nb, (uint8_t *)w->qs, (uint16_t *)w->d);
  } else if (w->dtype == HIPQ_Q4_K) {
    const int nb = (int)(w->K / 256);
    const int64_t total = w->N * nb;
    hipq::launch_kernel("relayout_q4_K", relayout_q4_K, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, src,
                       x8, w->N, nb, (uint8_t *)w->qs, (uint8_t *)w->hdr);
  } else {
    const int64_t total = w->N * (w->K / 256);
    hipq::launch_kernel("relayout_q6_K", relayout_q6_K, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, src,
                       total, (uint8_t *)w->qs, (uint8_t *)w->qh, (int8_t *)w->sc,
                       (uint16_t *)w->d);
  }
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
