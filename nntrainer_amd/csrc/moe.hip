// SPDX-License-Identifier: Apache-2.0
/**
 * @file   moe.hip
 * @brief  Mixture-of-experts feed-forward block on gfx950: on-device routing,
 *         token sort by expert and one grouped launch per projection.
 *
 * Replaces MoELayer::incremental_forwarding and compute_expert_forward_no_critical
 * (Applications/CausalLM/layers/qwen_moe_layer.cpp:394-503, 332-392 in the
 * reference checkout), which loop over experts on the host and issue three
 * single-row matmuls per (token, expert) pair. Semantics kept:
 *   - probabilities: softmax over the E logits (row max subtracted, exp,
 *     division by the row sum; nntrainer/layers/acti_func.h:166-213);
 *   - top-k by descending probability (nntrainer/tensor/float_tensor.cpp:1108-1180),
 *     ties to the lower expert id; weights divided by their sum when renormalize;
 *   - per pair: h = (sigmoid(g) * g) * u with sigmoid evaluated in double and
 *     cast to float (acti_func.h:286-288, 400-405), o = h . Wdown, o * weight;
 *   - a token's contributions are added in ascending expert id
 *     (qwen_moe_layer.cpp:493-498).
 * Every (token, expert) activation is quantized with the row quantizer, as the
 * reference's M = 1 matmuls do.
 *
 * Launch plan (all on one stream, no host synchronisation; grids do not depend
 * on device data): router logits (optional) -> route -> sort of the pairs by
 * expert (one workgroup; count / scan / scatter kernels for very long chunks),
 * which also lists the work items (expert, chunk of its slots) -> quantize x ->
 * grouped gate+up product with fused SwiGLU over (column tiles x work items) ->
 * quantize h -> grouped down product scaled by the routing weight -> combine.
 * Q4_K experts whose rows fit the LDS run on the matrix cores, 8 to 32 tokens of
 * an expert per work item; the other formats and longer rows use the decode
 * GEMV's engine, four tokens per pass over an expert's weights. Both carry the
 * reference's bits for every single-row product. Chunks of 17 to a few dozen tokens
 * over many experts take a form without the sort (gate_up_self_kernel below): four
 * launches, one workgroup row per expert.
 */
#include "gemv_device.h"
#include "quantize_device.h"

namespace {

constexpr int RTOK = 4; /* tokens sharing one pass over an expert's weight rows */

struct MoeBufs {
  float *logits;
  int32_t *idx;
  float *wgt;
  int *counts, *offsets, *cursor;
  int *slot_pair; /* pair (token * topk + k) of each slot */
  int *tok_slots; /* [T][topk]: a token's slots in ascending expert id */
  int *items;     /* [0] = number of work items, then (expert, first slot) per item */
  float *h;       /* [P][I] by slot */
  float *contrib; /* [P][H] by slot */
  void *xq_mem, *hq_mem;
  const int32_t *idx_used = nullptr; /* where this call's routing wrote the expert ids */
};

size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

size_t carve(const hipq_moe_desc &d, int is_k, uint8_t *base, MoeBufs *b) {
  const size_t T = d.tokens, H = d.hidden, I = d.intermediate, E = d.experts, P = T * d.topk;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    size_t at = o;
    o += up256(bytes);
    return base ? base + at : (uint8_t *)nullptr;
  };
  uint8_t *p;
  p = take(T * E * 4);
  if (b) b->logits = (float *)p;
  p = take(P * 4);
  if (b) b->idx = (int32_t *)p;
  p = take(P * 4);
  if (b) b->wgt = (float *)p;
  p = take(E * 4);
  if (b) b->counts = (int *)p;
  p = take((E + 1) * 4);
  if (b) b->offsets = (int *)p;
  p = take(E * 4);
  if (b) b->cursor = (int *)p;
  p = take(P * 4);
  if (b) b->slot_pair = (int *)p;
  p = take(P * 4);
  if (b) b->tok_slots = (int *)p;
  p = take((2 * (E + P) + 2) * 4);
  if (b) b->items = (int *)p;
  p = take(P * I * 4);
  if (b) b->h = (float *)p;
  p = take(P * H * 4);
  if (b) b->contrib = (float *)p;
  p = take(qact_bytes(is_k, T, H));
  if (b) b->xq_mem = p;
  p = take(qact_bytes(is_k, P, I));
  if (b) b->hq_mem = p;
  return o;
}

/* logits[t][e] = sum_h x[t][h] * Wr[h][e] (+ bias[e], added after the sum as the reference
 * adds it to the finished product, gpt_oss_moe_layer.cpp:500-503): one thread per logit, one
 * chain over h. For expert counts that are no multiple of four. */
__global__ __launch_bounds__(256) void router_logits_scalar_kernel(const float *__restrict__ x,
                                                                   const float *__restrict__ wr, int H,
                                                                   int E, const float *__restrict__ bias,
                                                                   float *__restrict__ logits) {
  const int t = blockIdx.x;
  const float *xt = x + (size_t)t * H;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    float acc = 0.f;
    for (int h = 0; h < H; ++h) acc = fmaf(xt[h], wr[(size_t)h * E + e], acc);
    logits[(size_t)t * E + e] = bias ? acc + bias[e] : acc;
  }
}

/* The same for E % 4 == 0, which is every model on this path. The single chain is bound by the
 * latency of its loads (2048 dependent rounds: 28 us for ONE token against 24 us for the rest of
 * the block), and one workgroup per token by what one CU can pull out of the cache (Wr is 1 MB:
 * 12 us). Here a workgroup takes sixteen experts (64 bytes of every row of Wr) and up to four
 * tokens, whose rows of x it first copies to LDS. Four lanes read a row's 64 bytes, sixteen rows
 * an instruction (sixteen half lines, not sixty-four separate ones), the four wavefronts take the
 * rows in turn, thirty-two loads are in flight (issued before the rows of x are copied) and each is
 * used for all the tokens. The partial sums
 * meet in a fixed order: over the sixteen row lanes by exchanges, over the wavefronts through LDS.
 * The matrix is read by E / 16 CUs side by side, each its own columns. (The reference's order of
 * the sum is its BLAS library's and not specified.) */
constexpr int ROUTER_TB = 4; /* tokens per workgroup, at most */
constexpr size_t router_lds_bytes(int tb_n, int H) { return ((size_t)tb_n * H + 256 * (size_t)tb_n) * sizeof(float); }
template <int TBN> /* tokens of this workgroup: 1, 2 or 4 */
__global__ __launch_bounds__(256) void router_logits_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ wr, int T, int H,
                                                            int E, const float *__restrict__ bias,
                                                            float *__restrict__ logits) {
  extern __shared__ __attribute__((aligned(16))) float router_x[]; /* [token][H], then the partial sums */
  constexpr int JU = 8; /* groups of four rows a lane has in flight: thirty-two loads (all of H = 2048 at once) */
  const int t0 = blockIdx.y * TBN;
  float *part = router_x + TBN * H; /* [wavefront 4][row of 16 lanes 4][token][16 experts] */
  const int e4n = E >> 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane >> 2, q = lane & 3;
  const int c = min((int)blockIdx.x * 4 + q, e4n - 1); /* columns past the end repeat the last; not stored */
  /* this lane's rows: h = 256 j + 64 wave + 4 r + i, i = 0 .. 3 (its x values are one 128-bit LDS read) */
  int h = 64 * wave + 4 * r;
  const bool whole = (H & 255) == 0; /* then a group of rows 256 j .. 256 j + 255 is in or out as one (uniform) */
  float4 w[JU][4];
  auto load_w = [&](int h0) {
    if (whole) {
      const float4 *p = (const float4 *)wr + c + (size_t)h0 * e4n;
#pragma unroll
      for (int j = 0; j < JU; ++j)
        if (256 * j + (h0 & ~255) < H) {
#pragma unroll
          for (int i = 0; i < 4; ++i) w[j][i] = p[(size_t)(256 * j + i) * e4n];
        }
    } else {
#pragma unroll
      for (int j = 0; j < JU; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) w[j][i] = ((const float4 *)wr + c)[(size_t)min(h0 + 256 * j + i, H - 1) * e4n];
    }
  };
  /* the first rows of Wr are on their way while the tokens' rows of x go to LDS, 2 * TBN loads of a lane at a
   * time (one after the other they cost a round trip each: 2.4 us for four rows of 2048) */
  load_w(h);
  const float *xrow[TBN];
#pragma unroll
  for (int tb = 0; tb < TBN; ++tb) xrow[tb] = x + (size_t)min(t0 + tb, T - 1) * H;
  for (int hx0 = threadIdx.x * 4; hx0 < H; hx0 += 2048) { /* H % 4 == 0 */
    float4 v[TBN][2];
#pragma unroll
    for (int tb = 0; tb < TBN; ++tb)
#pragma unroll
      for (int u = 0; u < 2; ++u) v[tb][u] = *(const float4 *)(xrow[tb] + min(hx0 + 1024 * u, H - 4));
#pragma unroll
    for (int tb = 0; tb < TBN; ++tb)
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (hx0 + 1024 * u < H) *(float4 *)(router_x + tb * H + hx0 + 1024 * u) = v[tb][u];
  }
  __syncthreads();
  float acc[TBN][4];
#pragma unroll
  for (int tb = 0; tb < TBN; ++tb) acc[tb][0] = acc[tb][1] = acc[tb][2] = acc[tb][3] = 0.f;
  for (; h < H; h += 256 * JU) {
#pragma unroll
    for (int j = 0; j < JU; ++j) {
      if (h + 256 * j < H) { /* H % 4 == 0: the four rows are in or out together */
#pragma unroll
        for (int tb = 0; tb < TBN; ++tb) {
          const float4 xv = *(const float4 *)(router_x + tb * H + h + 256 * j);
          const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            acc[tb][0] = fmaf(xs[i], w[j][i].x, acc[tb][0]);
            acc[tb][1] = fmaf(xs[i], w[j][i].y, acc[tb][1]);
            acc[tb][2] = fmaf(xs[i], w[j][i].z, acc[tb][2]);
            acc[tb][3] = fmaf(xs[i], w[j][i].w, acc[tb][3]);
          }
        }
      }
    }
    if (h + 256 * JU < H) load_w(h + 256 * JU);
  }
  /* The partial sums meet in a fixed order: the four lanes of a column quarter inside a row of sixteen lanes by
   * two shifted adds (lanes 12 .. 15 of the row then hold the row's sums), the sixteen rows of the workgroup
   * through LDS. (Exchanges across the whole wavefront, four a value, took 2.2 us of this kernel's 8.) */
  const int row16 = lane >> 4;
#pragma unroll
  for (int tb = 0; tb < TBN; ++tb) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v = acc[tb][j];
      v += hipq_dpp_f<0x114>(v); /* row_shr:4 */
      v += hipq_dpp_f<0x118>(v); /* row_shr:8 */
      if ((lane & 12) == 12) part[((wave * 4 + row16) * TBN + tb) * 16 + q * 4 + j] = v;
    }
  }
  __syncthreads();
  if (threadIdx.x < TBN * 16) {
    const int tb = threadIdx.x >> 4, el = threadIdx.x & 15, e = blockIdx.x * 16 + el;
    if (t0 + tb < T && e < E) {
      float sum = part[tb * 16 + el];
      for (int p = 1; p < 16; ++p) sum += part[(p * TBN + tb) * 16 + el];
      logits[(size_t)(t0 + tb) * E + e] = bias ? sum + bias[e] : sum;
    }
  }
}

/* Routing of token t by one wavefront: softmax, top-k, optional renormalisation, into registers:
 * lane kk < topk ends up with the kk-th choice's expert and weight. */
template <int MAXV> /* logits per lane: E <= 64 * MAXV */
__device__ __forceinline__ void route_token_regs(const float *__restrict__ logits, int t, int E, int topk,
                                                 int renorm, int &myi, float &myw) {
  const int lane = threadIdx.x & 63;
  float p[MAXV];
  const float *lg = logits + (size_t)t * E;
  float mx = -INFINITY;
  /* every lane's loads at once and unconditionally (a lane without an expert reads the last one's): behind
   * a condition each load is a round trip of its own */
#pragma unroll
  for (int i = 0; i < MAXV; ++i) p[i] = lg[min(lane + 64 * i, E - 1)];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    if (lane + 64 * i >= E) p[i] = -INFINITY;
    if (64 * i < E) mx = fmaxf(mx, p[i]);
  }
  mx = hipq_wave_max(mx);
  float sum = 0.f;
  /* the guards on 64 * i are uniform: rounds past E cost nothing (the double exponential is a few hundred
   * instructions) */
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    if (64 * i < E) {
      const int e = lane + 64 * i;
      p[i] = e < E ? (float)exp((double)(p[i] - mx)) : 0.f;
      sum += p[i];
    }
  }
  sum = hipq_wave_sum(sum);
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int e = lane + 64 * i;
    p[i] = (64 * i < E && e < E) ? __fdiv_rn(p[i], sum) : -1.f; /* -1: never selected */
    /* A NaN among the logits makes every probability NaN, which no comparison below
     * would ever select: the stored index would lie outside [0, E) and the kernels
     * behind index tables with it. Such values count as 0, so the selection still
     * returns topk distinct experts (the reference's partial_sort always does). */
    if (!(p[i] == p[i])) p[i] = 0.f;
  }
  float ksum = 0.f;
  myw = 0.f; /* lane kk keeps the kk-th weight */
  myi = 0;
  for (int kk = 0; kk < topk; ++kk) {
    float bv = -2.f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int e = lane + 64 * i;
      if (64 * i < E && p[i] > bv) { /* ascending e within the lane: first maximum wins */
        bv = p[i];
        bi = e;
      }
    }
    /* the wavefront's maximum, then the lowest expert id that holds it: mostly one lane's */
    const float mxv = hipq_wave_max(bv);
    const unsigned long long holders = __ballot(bv == mxv);
    const int cand = __popcll(holders) == 1 ? __builtin_amdgcn_readlane(bi, __ffsll((long long)holders) - 1)
                                            : hipq_wave_min_i(bv == mxv ? bi : 0x7fffffff);
    bv = mxv;
    bi = cand;
    /* every lane now agrees on (bv, bi); retire it in its owner */
    if ((bi & 63) == lane) {
#pragma unroll
      for (int i = 0; i < MAXV; ++i)
        if (i == (bi >> 6)) p[i] = -1.f;
    }
    ksum += bv;
    if (lane == kk) {
      myw = bv;
      myi = bi;
    }
  }
  if (renorm) myw = __fdiv_rn(myw, ksum);
}

/* The SET of token 0's topk experts without the exponentials and without a selection round per expert:
 * mask[i] bit l = expert 64 i + l is one of them. Returns false when the shortcut cannot promise the set
 * of route_token_regs, and the caller runs that. The probability p = fdiv(float(exp(double(v))), sum) with
 * v = logit - max <= 0 is monotone in v, so the sets can differ only if the topk-th and the next
 * probability round to the same float while their logits differ (the tie then goes to the lower expert
 * id). With v_topk - v_next > 1e-6 the two exponentials differ by more than eight float spacings and stay
 * apart through both roundings; with v_topk > -75 nothing underflows. A NaN or an infinite maximum among
 * the logits, and equal values on the two sides of the cut, take the full routine as well.
 * The topk-th largest v is the topk-th smallest magnitude |v| (as an integer: the bits of a float order
 * like its magnitude), found one bit at a time from counts over the wavefront: 31 steps of two compares
 * and a few scalar instructions, where a round of selection per expert is two dependent reductions over
 * the wavefront each (2.6 us for eight experts of 128, against 0.7 us). */
template <int MAXV>
__device__ __forceinline__ bool topk_set_fast(const float *__restrict__ lg, int E, int topk,
                                              unsigned long long (&mask)[MAXV]) {
  const int lane = threadIdx.x & 63;
  float v[MAXV];
  float mx = -INFINITY;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) v[i] = lg[min(lane + 64 * i, E - 1)]; /* all loads at once, see route_token_regs */
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    if (lane + 64 * i >= E) v[i] = -INFINITY;
    if (64 * i < E) {
      nan |= !(v[i] == v[i]);
      mx = fmaxf(mx, v[i]);
    }
  }
  if (__ballot(nan)) return false;
  mx = hipq_wave_max(mx);
  if (!(fabsf(mx) < INFINITY)) return false; /* uniform: an infinite logit makes differences undefined */
  int mag[MAXV]; /* |logit - max| as an integer; no expert's: beyond every float */
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int e = lane + 64 * i;
    mag[i] = (64 * i < E && e < E) ? (int)(__float_as_uint(v[i] - mx) & 0x7fffffffu) : 0x7fffffff;
  }
  auto count_le = [&](int t) {
    int n = 0;
#pragma unroll
    for (int i = 0; i < MAXV; ++i)
      if (64 * i < E) n += __popcll(__ballot(mag[i] <= t));
    return n;
  };
  int cut = 0; /* the smallest t with topk magnitudes <= t */
  for (int bit = 30; bit >= 0; --bit)
    if (count_le(cut | ((1 << bit) - 1)) < topk) cut |= 1 << bit;
  if (count_le(cut) != topk) return false; /* equal values across the cut: the tie rule decides (uniform) */
  int beyond = 0x7fffffff;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) beyond = min(beyond, mag[i] > cut ? mag[i] : 0x7fffffff);
  beyond = hipq_wave_min_i(beyond); /* the next magnitude, or 0x7fffffff when every expert is selected */
#pragma unroll
  for (int i = 0; i < MAXV; ++i) mask[i] = 64 * i < E ? __ballot(mag[i] <= cut) : 0ull;
  const float v_cut = __uint_as_float((uint32_t)cut);
  if (!(v_cut < 75.f)) return false;
  return beyond == 0x7fffffff || __uint_as_float((uint32_t)beyond) - v_cut > 1e-6f;
}

/* expert number `item` of the set in ascending id */
template <int MAXV> __device__ __forceinline__ int nth_of_set(const unsigned long long (&mask)[MAXV], int item) {
  int e = 0;
  bool found = false;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int c = __popcll(mask[i]);
    if (!found && item < c) {
      unsigned long long m = mask[i];
      for (int j = 0; j < item; ++j) m &= m - 1; /* drop the item lowest */
      e = 64 * i + __ffsll((long long)m) - 1;
      found = true;
    }
    if (!found) item -= c;
  }
  return e;
}

/* the rank of lane kk's expert among the token's topk, ascending expert id (lanes below topk) */
__device__ __forceinline__ int rank_by_expert(int myi, int topk) {
  int r = 0;
  for (int j = 0; j < topk; ++j) r += __builtin_amdgcn_readlane(myi, j) < myi;
  return r;
}

/* ... and written out */
template <int MAXV>
__device__ __forceinline__ void route_token(const float *__restrict__ logits, int t, int E, int topk,
                                            int renorm, int32_t *idx, float *wgt, int *by_expert = nullptr) {
  const int lane = threadIdx.x & 63;
  int myi;
  float myw;
  route_token_regs<MAXV>(logits, t, E, topk, renorm, myi, myw);
  if (by_expert) {
    /* the token's pairs in ascending expert id, the order in which its contributions are added
     * (tok_slots, for the forms that number the rows of h by pair instead of by sorted slot) */
    const int r = rank_by_expert(myi, topk);
    if (lane < topk) by_expert[(size_t)t * topk + r] = t * topk + lane;
  }
  if (lane < topk) {
    idx[(size_t)t * topk + lane] = myi;
    wgt[(size_t)t * topk + lane] = myw;
  }
}

template <int MAXV>
__global__ __launch_bounds__(256) void route_kernel(const float *__restrict__ logits, int T, int E,
                                                    int topk, int renorm, int32_t *__restrict__ idx,
                                                    float *__restrict__ wgt) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return; /* uniform per wavefront */
  route_token<MAXV>(logits, t, E, topk, renorm, idx, wgt);
}

/* Where the slot of pair i goes in tok_slots: a token's slots in ascending expert
 * id, the order in which its contributions are added. */
__device__ __forceinline__ int rank_in_token(const int32_t *idx, int i, int topk) {
  const int t = i / topk;
  const int e = idx[i];
  int r = 0;
  for (int j = 0; j < topk; ++j) r += idx[t * topk + j] < e;
  return t * topk + r;
}

/* The kernels below index tables of E entries with the expert ids that route_token wrote in
 * the same call: it always stores topk distinct ids in [0, E) (topk <= E is checked at the
 * boundary; a NaN probability counts as 0 and is still selectable), so the ids need no
 * further range check here.
 *
 * Count, scan and scatter of the (token, k) pairs by expert in one workgroup of
 * 1024 threads: the sort of a decode step or a short prefill chunk is a few thousand
 * pairs, and four tiny launches would cost more than the work. E <= 1024. */
__device__ __forceinline__ void sort_pairs(const int32_t *idx, int P, int E, int topk, int *__restrict__ offsets,
                                           int *__restrict__ slot_pair, int *__restrict__ tok_slots, int chunk,
                                           int *__restrict__ items) {
  __shared__ int cnt[1024];
  __shared__ int off[1024];
  __shared__ int wsum[16];
  __shared__ int nitems;
  const int t = threadIdx.x;
  cnt[t] = 0;
  if (t == 0) nitems = 0;
  __syncthreads();
  for (int i = t; i < P; i += 1024) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  /* exclusive scan over the 1024 slots: prefix sums inside each wavefront, then the
   * sixteen wavefront totals */
  const int own = cnt[t];
  int winc = own;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int v = __shfl_up(winc, d, 64);
    if ((t & 63) >= d) winc += v;
  }
  if ((t & 63) == 63) wsum[t >> 6] = winc;
  __syncthreads();
  int wbase = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) wbase += w < (t >> 6) ? wsum[w] : 0;
  const int excl = wbase + winc - own;
  if (t < E) offsets[t] = excl;
  if (t == E - 1) offsets[E] = excl + own;
  /* work items of the expert kernels: an expert's slots in chunks. A wavefront
   * numbers its experts' chunks with a prefix sum and takes its range of the list
   * with one atomic (the order of the wavefronts' ranges does not matter). */
  if (chunk > 0) {
    const int nch = t < E ? (own + chunk - 1) / chunk : 0;
    int incl = nch;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int v = __shfl_up(incl, d, 64);
      if ((t & 63) >= d) incl += v;
    }
    int base = 0;
    if ((t & 63) == 63 && incl > 0) base = atomicAdd(&nitems, incl);
    base = __shfl(base, 63, 64);
    const int at = base + incl - nch;
    for (int c = 0; c < nch; ++c) {
      items[2 + 2 * (at + c)] = t;
      items[3 + 2 * (at + c)] = excl + c * chunk;
    }
    __syncthreads();
    if (t == 0) items[0] = nitems;
  }
  off[t] = excl;
  cnt[t] = 0;
  __syncthreads();
  for (int i = t; i < P; i += 1024) {
    const int e = idx[i];
    const int slot = off[e] + atomicAdd(&cnt[e], 1);
    slot_pair[slot] = i;
    tok_slots[rank_in_token(idx, i, topk)] = slot;
  }
}

__global__ __launch_bounds__(1024) void sort_pairs_kernel(const int32_t *__restrict__ idx, int P, int E, int topk,
                                                          int *__restrict__ offsets, int *__restrict__ slot_pair,
                                                          int *__restrict__ tok_slots, int chunk,
                                                          int *__restrict__ items) {
  sort_pairs(idx, P, E, topk, offsets, slot_pair, tok_slots, chunk, items);
}

/* Routing and sort of up to 16 tokens (a decode step) in one launch: a wavefront
 * routes each token, then the workgroup sorts the pairs it has just written. */
template <int MAXV>
__global__ __launch_bounds__(1024) void route_sort_kernel(const float *__restrict__ logits, int T, int E, int topk,
                                                          int renorm, int32_t *idx, float *wgt,
                                                          int *__restrict__ offsets, int *__restrict__ slot_pair,
                                                          int *__restrict__ tok_slots, int chunk,
                                                          int *__restrict__ items) {
  const int t = threadIdx.x >> 6;
  if (t < T) route_token<MAXV>(logits, t, E, topk, renorm, idx, wgt);
  __syncthreads(); /* orders the routing's stores before the sort's loads */
  sort_pairs(idx, T * topk, E, topk, offsets, slot_pair, tok_slots, chunk, items);
}

/* The rows of x quantized for the matrix-core expert kernels, in the same launch as
 * the routing (neither needs the other): workgroups 0 .. route_blocks - 1 route (or
 * route and sort, with 1024 threads), the others quantize one super-block per
 * wavefront. */
struct XQuant {
  const float *x;
  int64_t n_sb; /* T * H / 256 */
  int nsb;
  int8_t *q;
  float *d;
  uint16_t *amin;
};
__device__ __forceinline__ void quantize_x(const XQuant &xq, int T, int block) {
  const int64_t sb = (int64_t)block * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (sb >= xq.n_sb) return; /* uniform per wavefront */
  hipq_quantize_q8_K_wave<Q8K_ROWMMA>(xq.x, T, sb, xq.nsb, (int64_t)xq.nsb * 256, 0, xq.q, xq.d, nullptr, nullptr,
                                      xq.amin, nullptr, nullptr);
}

template <int MAXV>
__global__ __launch_bounds__(256) void route_quantize_kernel(const float *__restrict__ logits, int T, int E,
                                                             int topk, int renorm, int32_t *__restrict__ idx,
                                                             float *__restrict__ wgt, int route_blocks,
                                                             XQuant xq, int *__restrict__ by_expert) {
  if ((int)blockIdx.x >= route_blocks) {
    quantize_x(xq, T, blockIdx.x - route_blocks);
    return;
  }
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return; /* uniform per wavefront */
  route_token<MAXV>(logits, t, E, topk, renorm, idx, wgt, by_expert);
}

template <int MAXV>
__global__ __launch_bounds__(1024) void route_sort_quantize_kernel(
  const float *__restrict__ logits, int T, int E, int topk, int renorm, int32_t *idx, float *wgt,
  int *__restrict__ offsets, int *__restrict__ slot_pair, int *__restrict__ tok_slots, int chunk,
  int *__restrict__ items, XQuant xq) {
  if (blockIdx.x > 0) {
    quantize_x(xq, T, blockIdx.x - 1);
    return;
  }
  const int t = threadIdx.x >> 6;
  if (t < T) route_token<MAXV>(logits, t, E, topk, renorm, idx, wgt);
  __syncthreads(); /* orders the routing's stores before the sort's loads */
  sort_pairs(idx, T * topk, E, topk, offsets, slot_pair, tok_slots, chunk, items);
}

__global__ void fill_int_kernel(int *p, int n, int v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ void count_kernel(const int32_t *__restrict__ idx, int P, int *__restrict__ counts) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < P) atomicAdd(&counts[idx[i]], 1);
}

__global__ void scan_kernel(const int *__restrict__ counts, int E, int *__restrict__ offsets,
                            int *__restrict__ cursor, int chunk, int *__restrict__ items) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int acc = 0, n = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      if (chunk > 0)
        for (int c = 0; c < counts[e]; c += chunk) {
          items[2 + 2 * n] = e;
          items[3 + 2 * n] = acc + c;
          ++n;
        }
      acc += counts[e];
      cursor[e] = 0;
    }
    offsets[E] = acc;
    items[0] = n;
  }
}

__global__ void scatter_kernel(const int32_t *__restrict__ idx, int P, int topk,
                               const int *__restrict__ offsets, int *__restrict__ cursor,
                               int *__restrict__ slot_pair, int *__restrict__ tok_slots) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  const int e = idx[i];
  const int slot = offsets[e] + atomicAdd(&cursor[e], 1);
  slot_pair[slot] = i;
  tok_slots[rank_in_token(idx, i, topk)] = slot;
}

__device__ __forceinline__ float silu_ref(float g) {
  /* sigmoid in double on the float-rounded exponential, as the reference */
  const float en = (float)exp((double)(-g));
  const float sig = (float)(1.0 / (1.0 + (double)en));
  return sig * g;
}

/* The activation between the projections and the bias of the down projection, by expert
 * variant (hipq_internal.h, MoeEpi). For the biased variant the value of column col of expert
 * e is (g / (1 + exp(-alpha g))) * (u + 1) with g and u the biased (and, for the cached layer,
 * clamped) products, in fp32 (gpt_oss_moe_layer.cpp:406-437; swiglu with alpha,
 * fallback_internal.cpp:425-432). */
__device__ __forceinline__ float moe_act(const hipq::MoeEpi &ep, int e, int I, int col, float g, float u) {
  if (ep.kind == 0) return silu_ref(g) * u;
  g = g + ep.gate_bias[(size_t)e * I + col];
  u = u + ep.up_bias[(size_t)e * I + col];
  if (ep.limit > 0.f) { /* the cached layer's clamps, gpt_oss_moe_layer_cached.cpp:497-507 */
    g = g < ep.limit ? g : ep.limit;
    u = u > -ep.limit ? u : -ep.limit;
    u = u < ep.limit ? u : ep.limit;
  }
  u = u + 1.f;
  return (g / (1.f + expf(-ep.alpha * g))) * u;
}
__device__ __forceinline__ float moe_out(const hipq::MoeEpi &ep, int e, int H, int col, float o, float w) {
  if (ep.kind != 0) o = o + ep.down_bias[(size_t)e * H + col];
  return o * w;
}

/* One group of G weight rows against the cached activations: phase 1 into the
 * wavefront's LDS records, phase 2 fp32 chains, result of this lane's chain. */
template <typename E>
__device__ __forceinline__ GemvOut run_group(const typename E::Wts &W, const typename E::Act &A,
                                             const int (&arow)[RTOK], int K, uint32_t *lds) {
  typename E::Chain c = E::begin(arow, 0);
  E::compute(W, A, K, lds);
  hipq_wave_lds_sync();
  E::chain(c, K, lds);
  hipq_wave_lds_sync();
  return E::finish(c);
}

/* h[slot][col] = silu(x_tok . Wgate[e][col]) * (x_tok . Wup[e][col])
 *
 * A workgroup serves one expert; each wavefront owns CPW groups of G columns.
 * Per group of RTOK tokens it loads their quantized activations once, then walks
 * its column groups with the gate rows and the up rows of a group as two work
 * items; the weight loads of the next item are always in flight while the current
 * one is computed. Requires K <= KC (one chunk). */
template <int DT, int T, int KC, int G, int CPW>
__global__ __launch_bounds__(256) void gate_up_kernel(const WView *__restrict__ views, int E_,
                                                      QView xq, const int *__restrict__ offsets,
                                                      const int *__restrict__ slot_pair, int topk,
                                                      int I, float *__restrict__ h, hipq::MoeEpi ep) {
  typedef GemvCore<DT, T, RTOK, G, false, KC> E;
  extern __shared__ uint32_t moe_lds[];
  const int e = blockIdx.y;
  const int begin = offsets[e], end = offsets[e + 1];
  if (begin == end) return;
  const WView wg = views[e], wu = views[E_ + e];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = moe_lds + wave * GemvLds<DT, RTOK, G, false>::DWORDS;
  const int cbase = (blockIdx.x * 4 + wave) * CPW * G;
  if (cbase >= I) return; /* uniform per wavefront; the syncs below are wavefront-local */
  const int K = wg.K;
  for (int s0 = begin; s0 < end; s0 += RTOK) {
    int arow[RTOK];
#pragma unroll
    for (int r = 0; r < RTOK; ++r) {
      const int slot = min(s0 + r, end - 1);
      arow[r] = slot_pair[slot] / topk; /* token of the pair */
    }
    typename E::Act A;
    E::load_act(A, xq, arow, 0, K);
    typename E::Wts Wg, Wu;
    E::load_w(Wg, wg, cbase, 0, K);
#pragma unroll
    for (int cg = 0; cg < CPW; ++cg) {
      const int col0 = cbase + cg * G;
      if (col0 >= I) break; /* uniform */
      E::load_w(Wu, wu, col0, 0, K);
      const GemvOut g = run_group<E>(Wg, A, arow, K, lds);
      if (cg + 1 < CPW && col0 + G < I) E::load_w(Wg, wg, col0 + G, 0, K);
      const GemvOut u = run_group<E>(Wu, A, arow, K, lds);
      if (g.valid && col0 + g.g < I && s0 + g.r < end)
        h[(size_t)(s0 + g.r) * I + col0 + g.g] = moe_act(ep, e, I, col0 + g.g, g.v, u.v);
    }
  }
}

/* contrib[slot][col] = (h_slot . Wdown[e][col]) * weight(pair); same structure */
template <int DT, int T, int KC, int G, int CPW>
__global__ __launch_bounds__(256) void down_kernel(const WView *__restrict__ views, int E_, QView hq,
                                                   const int *__restrict__ offsets,
                                                   const int *__restrict__ slot_pair,
                                                   const float *__restrict__ wgt, int H,
                                                   float *__restrict__ contrib, hipq::MoeEpi ep) {
  typedef GemvCore<DT, T, RTOK, G, false, KC> E;
  extern __shared__ uint32_t moe_lds[];
  const int e = blockIdx.y;
  const int begin = offsets[e], end = offsets[e + 1];
  if (begin == end) return;
  const WView wd = views[2 * E_ + e];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = moe_lds + wave * GemvLds<DT, RTOK, G, false>::DWORDS;
  const int cbase = (blockIdx.x * 4 + wave) * CPW * G;
  if (cbase >= H) return;
  const int K = wd.K;
  for (int s0 = begin; s0 < end; s0 += RTOK) {
    int arow[RTOK];
#pragma unroll
    for (int r = 0; r < RTOK; ++r) arow[r] = min(s0 + r, end - 1); /* hq rows are slots */
    typename E::Act A;
    E::load_act(A, hq, arow, 0, K);
    typename E::Wts W[2];
    E::load_w(W[0], wd, cbase, 0, K);
#pragma unroll
    for (int cg = 0; cg < CPW; ++cg) {
      const int col0 = cbase + cg * G;
      if (col0 >= H) break;
      if (cg + 1 < CPW && col0 + G < H) E::load_w(W[(cg + 1) & 1], wd, col0 + G, 0, K);
      const GemvOut o = run_group<E>(W[cg & 1], A, arow, K, lds);
      if (o.valid && col0 + o.g < H && s0 + o.r < end)
        contrib[(size_t)(s0 + o.r) * H + col0 + o.g] = moe_out(ep, e, H, col0 + o.g, o.v, wgt[slot_pair[s0 + o.r]]);
    }
  }
}

/* The same two products for rows longer than one chunk (K > 4096): one engine call
 * per column group, no cross-group prefetch. */
template <int DT>
__global__ __launch_bounds__(256) void gate_up_long_kernel(const WView *__restrict__ views, int E_,
                                                           QView xq, const int *__restrict__ offsets,
                                                           const int *__restrict__ slot_pair,
                                                           int topk, int I, float *__restrict__ h,
                                                           hipq::MoeEpi ep) {
  constexpr int G = 2;
  extern __shared__ uint32_t moe_lds[];
  const int e = blockIdx.y;
  const int begin = offsets[e], end = offsets[e + 1];
  if (begin == end) return;
  const WView wg = views[e], wu = views[E_ + e];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = moe_lds + wave * GemvLds<DT, RTOK, G, false>::DWORDS;
  const int col0 = (blockIdx.x * 4 + wave) * G;
  for (int s0 = begin; s0 < end; s0 += RTOK) {
    int arow[RTOK];
#pragma unroll
    for (int r = 0; r < RTOK; ++r) {
      const int slot = min(s0 + r, end - 1);
      arow[r] = slot_pair[slot] / topk;
    }
    const GemvOut g = gemv_engine<DT, 64, RTOK, G, false>(wg, col0, xq, arow, 0, lds);
    const GemvOut u = gemv_engine<DT, 64, RTOK, G, false>(wu, col0, xq, arow, 0, lds);
    if (g.valid && col0 + g.g < I && s0 + g.r < end)
      h[(size_t)(s0 + g.r) * I + col0 + g.g] = moe_act(ep, e, I, col0 + g.g, g.v, u.v);
  }
}

template <int DT>
__global__ __launch_bounds__(256) void down_long_kernel(const WView *__restrict__ views, int E_,
                                                        QView hq, const int *__restrict__ offsets,
                                                        const int *__restrict__ slot_pair,
                                                        const float *__restrict__ wgt, int H,
                                                        float *__restrict__ contrib, hipq::MoeEpi ep) {
  constexpr int G = 2;
  extern __shared__ uint32_t moe_lds[];
  const int e = blockIdx.y;
  const int begin = offsets[e], end = offsets[e + 1];
  if (begin == end) return;
  const WView wd = views[2 * E_ + e];
  const int wave = threadIdx.x >> 6;
  uint32_t *lds = moe_lds + wave * GemvLds<DT, RTOK, G, false>::DWORDS;
  const int col0 = (blockIdx.x * 4 + wave) * G;
  for (int s0 = begin; s0 < end; s0 += RTOK) {
    int arow[RTOK];
#pragma unroll
    for (int r = 0; r < RTOK; ++r) arow[r] = min(s0 + r, end - 1);
    const GemvOut o = gemv_engine<DT, 64, RTOK, G, false>(wd, col0, hq, arow, 0, lds);
    if (o.valid && col0 + o.g < H && s0 + o.r < end)
      contrib[(size_t)(s0 + o.r) * H + col0 + o.g] = moe_out(ep, e, H, col0 + o.g, o.v, wgt[slot_pair[s0 + o.r]]);
  }
}

/* ---- Q4_K experts on the matrix cores --------------------------------------------
 *
 * With a handful of tokens per expert the products above redo the nibble unpacking
 * per token group. Here a wavefront owns 32 weight rows and up to 32 tokens and
 * forms the 32 x 32 integer block sums of a super-block with
 * v_mfma_i32_32x32x32_i8: the tokens' Q8_K values are the row operand (from LDS,
 * staged once per workgroup), the weights the column operand, unpacked in registers
 * from the nibbles. A matrix step is one sub-block: lane (n, g) supplies weights
 * 16g .. 16g+15 of it for weight row n, even ones (low nibbles) in operand bytes
 * 0-7 and odd ones in bytes 8-15, and the quantizer stores every 16-value group of
 * the activations in that order; the step's sums take the sub-block's 6-bit scale
 * in an integer multiply-add. The mins go through one v_mfma_f32_32x32x16_f16 per
 * super-block with the sub-block sums split into two fp16-exact parts. Every
 * integer is exact and the fp32 chain per output is the single-row kernel's, so the
 * results carry the same bits:
 *   acc = fma(float(I), d * dA, acc); accm = fma(float(Im), dmin * dA, accm).
 *
 * The unit of work is an item of the list the pair sort writes: up to TC slots of
 * one expert. A workgroup takes one item and 128 (gate/up) or 256 (down) columns,
 * so an expert with more than TC tokens is served by several workgroups side by
 * side instead of one that walks its weights several times. */
typedef int mv2i __attribute__((ext_vector_type(2)));
typedef int mv4i __attribute__((ext_vector_type(4)));
typedef int mv16i __attribute__((ext_vector_type(16)));
typedef float mv16f __attribute__((ext_vector_type(16)));
typedef _Float16 mv8h __attribute__((ext_vector_type(8)));

/* LDS of a workgroup: the item's TC activation rows, padded so that the lanes of a
 * 128-bit read fall into different banks. */
struct XLds {
  int8_t *q;     /* [TC][K + 16] */
  uint8_t *amin; /* [TC][nsb][32 bytes] */
  float *dA;     /* [nsb][TC] */
  int *rows;     /* [TC] source rows of the item */
  int *pairs;    /* the item's (token, k) pairs, where the workgroup finds them itself (the forms without a sort) */
};
__host__ __device__ inline size_t xlds_bytes(int TC, int K) {
  const size_t b = (size_t)TC * (K + 16) + (size_t)TC * (K / 256) * 32 + (size_t)TC * (K / 256) * 4 + TC * 4;
  return (b + 255) & ~(size_t)255;
}
__device__ __forceinline__ XLds xlds_carve(unsigned char *base, int TC, int K) {
  XLds l;
  l.q = (int8_t *)base;
  l.amin = (uint8_t *)base + (size_t)TC * (K + 16);
  l.dA = (float *)(l.amin + (size_t)TC * (K / 256) * 32);
  l.rows = (int *)(l.dA + (size_t)TC * (K / 256));
  l.pairs = nullptr;
  return l;
}

/* Copy the item's nrows activation rows (l.rows, already in LDS) from the planes of a; the
 * other rows of the matrix operand keep whatever the LDS held: a row of the product depends on
 * its own activations only, and those rows are not stored. Loads are issued four at a time
 * before their stores so that their latencies overlap. */
template <int TC>
__device__ __forceinline__ void stage_rows(const XLds &l, const QView &a, int nrows) {
  const int K = a.K, nsb = K >> 8;
  const int cpr = K >> 4; /* 16-byte pieces per row */
  const int nt = blockDim.x;
  const int np = nrows * cpr;
  for (int c0 = threadIdx.x; c0 < np; c0 += 4 * nt) {
    mv4i v0, v1, v2, v3;
    int d0, d1, d2, d3;
    auto ld = [&](int u, mv4i &v, int &dst) {
      const int c = min(c0 + u * nt, np - 1);
      const int r = c / cpr, o = c - r * cpr;
      v = *(const mv4i *)(a.q + (size_t)l.rows[r] * K + o * 16);
      dst = r * (K + 16) + o * 16;
    };
    ld(0, v0, d0), ld(1, v1, d1), ld(2, v2, d2), ld(3, v3, d3);
    *(mv4i *)(l.q + d0) = v0;
    if (c0 + nt < np) *(mv4i *)(l.q + d1) = v1;
    if (c0 + 2 * nt < np) *(mv4i *)(l.q + d2) = v2;
    if (c0 + 3 * nt < np) *(mv4i *)(l.q + d3) = v3;
  }
  for (int c = threadIdx.x; c < nrows * nsb * 2; c += nt) {
    const int r = c / (nsb * 2), o = c - r * (nsb * 2);
    const mv4i v = *(const mv4i *)((const uint8_t *)a.bsum + ((size_t)l.rows[r] * nsb) * 32 + o * 16);
    *(mv4i *)(l.amin + ((size_t)r * nsb) * 32 + o * 16) = v;
  }
  for (int c = threadIdx.x; c < nrows * nsb; c += nt) {
    const int r = c / nsb, b = c - r * nsb;
    l.dA[b * TC + r] = a.d[(size_t)l.rows[r] * nsb + b];
  }
}

/* The weight stream. The experts' weights are stored by tiles of 32 rows: per tile
 * and super-block four 1 KB groups, group i holding for lane (n, g) the halves g
 * (weights 16g .. 16g+15) of sub-blocks 2i and 2i+1 of row n, then the 32 headers
 * (512 bytes), the super-blocks of a tile one behind the other. A wavefront's 128-bit
 * load i therefore reads 1 KB of consecutive memory (whole cache lines, marked
 * non-temporal), its stream over a tile is one run of consecutive memory, and every
 * lane receives exactly the bytes of its two matrix steps. The loads of the next super-block are in flight during the
 * arithmetic of the current one, also across tiles; nothing but the activations
 * occupies LDS, so the number of resident wavefronts is bounded by registers (four
 * per SIMD for TC = 8) and one launch holds all work items of a prefill chunk. */
constexpr int XPD = 1; /* super-blocks the loads run ahead of the arithmetic */
typedef __amdgpu_buffer_rsrc_t xrsrc_t;
struct XRegs {
  mv4i q[4];
  mv4i hd;
};

/* One super-block's terms for the NREG rows of a lane: the integer sum fi (as a float) with its factor
 * si = d * dA, and the mins' sum fm with its factor sm = dmin * dA. The caller adds them to its chains,
 * acc = fma(fi, si, acc) and accm = fma(fm, sm, accm), in super-block order. */
template <int TC, int NREG>
__device__ __forceinline__ void xr_sb_terms(const XRegs &W, const XLds &l, int K, int sb, int i32, int g,
                                            float (&fi)[NREG], float (&si)[NREG], float (&fm)[NREG],
                                            float (&sm)[NREG]) {
  const mv16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const mv16f zero16f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int nsb = K >> 8;
  const int row = i32 & (TC - 1);
  const int8_t *pa = l.q + row * (K + 16) + sb * 256 + g * 16;
  const mv8h amin = *(const mv8h *)(l.amin + (row * nsb + sb) * 32 + g * 16);
  mv4i dv[NREG / 4];
#pragma unroll
  for (int q4 = 0; q4 < NREG / 4; ++q4) dv[q4] = *(const mv4i *)(l.dA + sb * TC + 4 * g + q4 * 8);
  mv2i wq[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    wq[2 * i] = mv2i{W.q[i][0], W.q[i][1]};
    wq[2 * i + 1] = mv2i{W.q[i][2], W.q[i][3]};
  }
  const uint4 hd = make_uint4((uint32_t)W.hd[0], (uint32_t)W.hd[1], (uint32_t)W.hd[2], (uint32_t)W.hd[3]);
  const uint32_t s03 = hd.y & 0x3f3f3f3fu;
  const uint32_t s47 = hd.z & 0x3f3f3f3fu;
  int I[NREG];
#pragma unroll
  for (int r = 0; r < NREG; ++r) I[r] = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    /* weight 2i / 2i+1 of the lane's 16 in the low / high nibble of byte i: the even
     * ones become operand bytes 0-7, the odd ones bytes 8-15 (the activations'
     * 16-value groups are stored in that order) */
    const uint32_t x0 = (uint32_t)wq[j][0], x1 = (uint32_t)wq[j][1];
    const mv4i b = {(int)(x0 & HIPQ_M4), (int)(x1 & HIPQ_M4), (int)((x0 >> 4) & HIPQ_M4),
                    (int)((x1 >> 4) & HIPQ_M4)};
    const mv4i a8 = *(const mv4i *)(pa + j * 32);
    /* one result register for all steps: four wavefronts per SIMD hide the matrix
     * core's latency better than a second register (and a third wavefront) did */
    const mv16i D = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8, b, zero16, 0, 0, 0);
    const int scj = (int)(((j < 4 ? s03 : s47) >> (8 * (j & 3))) & 0xff);
#pragma unroll
    for (int r = 0; r < NREG; ++r) I[r] = __mul24(D[r], scj) + I[r];
  }
  const uint32_t mlo = (hd.w & 0x0f0f0f0fu) | ((hd.y >> 2) & 0x30303030u);
  const uint32_t mhi = ((hd.w >> 4) & 0x0f0f0f0fu) | ((hd.z >> 2) & 0x30303030u);
  mv8h bmin;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    bmin[j] = (_Float16)(float)((mlo >> (8 * j)) & 0xff);
    bmin[4 + j] = (_Float16)(float)((mhi >> (8 * j)) & 0xff);
  }
  const mv16f Sm = __builtin_amdgcn_mfma_f32_32x32x16_f16(amin, bmin, zero16f, 0, 0, 0);
  const float dw = hipq_h2f((uint16_t)(hd.x & 0xffff));
  const float dmin = hipq_h2f((uint16_t)(hd.x >> 16));
#pragma unroll
  for (int q4 = 0; q4 < NREG / 4; ++q4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int r = 4 * q4 + e;
      const float dA = __int_as_float(dv[q4][e]);
      fi[r] = (float)I[r];
      si[r] = dw * dA;
      fm[r] = Sm[r];
      sm[r] = dmin * dA;
    }
  }
}
template <int TC, int NREG>
__device__ __forceinline__ void xr_super_block(const XRegs &W, const XLds &l, int K, int sb, int i32, int g,
                                               float (&acc)[NREG], float (&accm)[NREG]) {
  float fi[NREG], si[NREG], fm[NREG], sm[NREG];
  xr_sb_terms<TC, NREG>(W, l, K, sb, i32, g, fi, si, fm, sm);
#pragma unroll
  for (int r = 0; r < NREG; ++r) {
    acc[r] = fmaf(fi[r], si[r], acc[r]);
    accm[r] = fmaf(fm[r], sm[r], accm[r]);
  }
}

/* A run of column tiles for one wavefront, the loads PD super-blocks ahead of the
 * arithmetic, also across tiles. tile_of(t, &view, &col0) names tile t; done(t, out)
 * receives its NREG results. */
template <int TC, int NREG, int PD, typename TileOf, typename Done, typename Pre>
__device__ __forceinline__ void xr_run(int ntile, const XLds &l, int K, TileOf tile_of, Done done, Pre pre) {
  constexpr int NB = PD + 1;
  const int lane = threadIdx.x & 63, i32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8;
  const int nv = ntile * nsb;
  /* the current tile (nibbles and headers of its super-blocks, EXPERT_TILE_BYTES each) as a
   * buffer descriptor in scalar registers: a load names the lane's offset and a scalar offset,
   * so no lane keeps or adds 64-bit addresses */
  xrsrc_t rq;
  int lt = 0, lsb = 0, issued = 0;
  auto open = [&](int t) {
    WView w;
    int c0;
    tile_of(t, w, c0);
    const int tile = c0 >> 5; /* c0 < N: rows past N are zero padding of the last tile */
    rq = __builtin_amdgcn_make_buffer_rsrc((void *)(w.qs + (size_t)tile * (size_t)(nsb * hipq::EXPERT_TILE_BYTES)), 0,
                                           nsb * hipq::EXPERT_TILE_BYTES, 0x00020000);
  };
  open(0);
  auto load = [&](XRegs &r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) /* non-temporal: every load instruction covers whole cache lines */
      r.q[i] = __builtin_bit_cast(
        mv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, lane * 16, lsb * hipq::EXPERT_TILE_BYTES + i * 1024, 2));
    r.hd = __builtin_bit_cast(
      mv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, 4096 + i32 * 16, lsb * hipq::EXPERT_TILE_BYTES, 2));
    if (++issued >= nv) return; /* uniform: the cursor stays on the last super-block */
    if (++lsb == nsb) {
      lsb = 0;
      open(++lt);
    }
  };
  /* Every step issues its loads, past the end of the stream those of the last
   * super-block again: a fixed number of loads is then in flight at each wait. */
  XRegs buf[NB];
#pragma unroll
  for (int p = 0; p < PD; ++p) load(buf[p]);
  pre(); /* the activations are staged while the first weights are on their way */
  int t = 0, sb = 0;
  float acc[NREG], accm[NREG];
  for (int v0 = 0; v0 < nv; v0 += NB) {
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int v = v0 + u;
      if (v < nv) {
        load(buf[(u + PD) % NB]);
        if (sb == 0) {
#pragma unroll
          for (int r = 0; r < NREG; ++r) acc[r] = accm[r] = 0.f;
        }
        xr_super_block<TC, NREG>(buf[u], l, K, sb, i32, g, acc, accm);
        if (++sb == nsb) {
          float out[NREG];
#pragma unroll
          for (int r = 0; r < NREG; ++r) out[r] = acc[r] - accm[r];
          done(t, out);
          sb = 0;
          ++t;
        }
      }
    }
  }
}

/* h[slot][col] = silu(x_tok . Wgate[e][col]) * (x_tok . Wup[e][col]) for one work
 * item. A wavefront forms the gate tile and then the up tile of its 32 columns
 * (128 columns per workgroup). With few items (decode, short chunks) that leaves
 * most of the chip idle, so the PAIRED form halves the stream per wavefront:
 * wavefronts 0-1 form the gate tiles and 2-3 the up tiles of 64 columns, and the
 * gate values cross through LDS. */
template <int TC, bool PAIRED>
__global__ __launch_bounds__(256, TC <= 8 ? 4 : TC <= 16 ? 2 : 1) void gate_up_mma_kernel(
  const WView *__restrict__ views, int E_, QView xq, const int *__restrict__ offsets,
  const int *__restrict__ items, const int *__restrict__ slot_pair, int topk, int I, float *__restrict__ h,
  hipq::MoeEpi ep) {
  constexpr int NREG = TC / 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char xmoe_lds[];
  const int item = blockIdx.y;
  if (item >= items[0]) return; /* uniform per workgroup */
  const int e = items[2 + 2 * item], s0 = items[3 + 2 * item];
  const int end = min(s0 + TC, offsets[e + 1]);
  const WView wg = views[e], wu = views[E_ + e];
  const int K = wg.K;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const XLds l = xlds_carve(xmoe_lds, TC, K);
  float *xch = (float *)(xmoe_lds + xlds_bytes(TC, K)); /* PAIRED: [2 tiles][NREG][64 lanes] */
  const int col0 = PAIRED ? (blockIdx.x * 2 + (wave & 1)) * 32 : (blockIdx.x * 4 + wave) * 32;
  const int first = PAIRED ? wave >> 1 : 0; /* 0: gate, 1: up */
  const uint64_t dqs = (uint64_t)wu.qs - (uint64_t)wg.qs;
  auto stage = [&]() {
    if (threadIdx.x < TC) l.rows[threadIdx.x] = slot_pair[min(s0 + (int)threadIdx.x, end - 1)] / topk;
    __syncthreads();
    stage_rows<TC>(l, xq, end - s0);
    __syncthreads();
  };
  float gate[NREG], up[NREG];
  auto store = [&]() {
    const int col = col0 + (lane & 31);
#pragma unroll
    for (int r = 0; r < NREG; ++r) {
      const int tok = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
      if (col < I && s0 + tok < end) h[(size_t)(s0 + tok) * I + col] = moe_act(ep, e, I, col, gate[r], up[r]);
    }
  };
  if (col0 >= I) { /* uniform per wavefront; it still takes part in the barriers */
    stage();
    if (PAIRED) __syncthreads();
    return;
  }
  xr_run<TC, NREG, XPD>(
    PAIRED ? 1 : 2, l, K,
    [&](int t, WView &w, int &c0) {
      const uint64_t isup = (uint64_t)0 - (uint64_t)((t + first) & 1);
      w.qs = (const uint8_t *)((uint64_t)wg.qs + (isup & dqs));
      w.hdr = nullptr; /* the headers follow the nibbles */
      w.N = wg.N;
      w.K = wg.K;
      c0 = col0;
    },
    [&](int t, const float(&out)[NREG]) {
      if (t + first == 0) {
#pragma unroll
        for (int r = 0; r < NREG; ++r) gate[r] = out[r];
      } else {
#pragma unroll
        for (int r = 0; r < NREG; ++r) up[r] = out[r];
      }
    },
    stage);
  /* the SwiGLU (a double-precision exponential) comes after the stream, when no
   * weights are held in registers any more */
  if (!PAIRED) store();
  if (PAIRED) {
    float *mine = xch + (wave & 1) * (NREG * 64) + lane;
    if (first == 0) {
#pragma unroll
      for (int r = 0; r < NREG; ++r) mine[r * 64] = gate[r];
    }
    __syncthreads();
    if (first == 1) {
#pragma unroll
      for (int r = 0; r < NREG; ++r) gate[r] = mine[r * 64];
      store();
    }
  }
}

/* floats of LDS one of (gate, up) needs for the terms of the second half of K in the one-token kernel */
__host__ __device__ constexpr int one_token_terms(int K) { return ((K >> 8) / 2 + 1) * 128; }

/* One token (a decode step), the routing inside the gate/up launch: every wavefront finds the
 * token's set of experts itself (the same arithmetic on the same logits, so all agree; without the
 * softmax's exponentials where topk_set_fast can promise the same set), the workgroup takes the
 * expert whose rank in ascending id is its blockIdx.y, quantizes the row of x into its LDS while
 * its first weights are on their way, and goes on as the paired form of gate_up_mma_kernel.
 * One workgroup more than the columns need routes the token in full and writes the routing's
 * outputs and the few table entries the down product and the combine read. One launch (7-8 us of
 * a block of 25) less than routing, sort and quantization as a launch of their own. */
template <int MAXV>
__global__ __launch_bounds__(256, 4) void gate_up_one_token_kernel(
  const float *__restrict__ logits, int E, int topk, int renorm, int32_t *__restrict__ idx, float *__restrict__ wgt,
  int *__restrict__ offsets, int *__restrict__ slot_pair, int *__restrict__ tok_slots, int *__restrict__ items,
  const float *__restrict__ x, const WView *__restrict__ views, int H, int I, float *__restrict__ h, hipq::MoeEpi ep) {
  constexpr int TC = 8, NREG = TC / 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char xmoe_lds[];
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  int myi;
  float myw;
  if (blockIdx.x == gridDim.x - 1) {
    /* the extra column of the grid: its first workgroup's first wavefront routes the token in full and
     * writes what the launches behind this one read; it multiplies nothing */
    if (blockIdx.y == 0 && wave == 0) {
      route_token_regs<MAXV>(logits, 0, E, topk, renorm, myi, myw);
      const int rank = rank_by_expert(myi, topk);
      if (lane < topk) {
        idx[lane] = myi;
        wgt[lane] = myw;
        slot_pair[rank] = lane; /* slots in ascending expert id; one token: pair = its k */
        tok_slots[rank] = rank;
        offsets[myi + 1] = rank + 1; /* the end of the expert's slots: all the later kernels read of offsets */
        items[2 + 2 * rank] = myi;
        items[3 + 2 * rank] = rank;
      }
      if (lane == 0) items[0] = topk;
    }
    return; /* uniform per workgroup */
  }
  /* this wavefront's share of the row of x is asked for first: it has arrived when the routing is done */
  constexpr int XPRE = 4; /* super-blocks a wavefront holds ahead: rows of up to 4096 values */
  const int nsb_x = H >> 8;
  float4 xpre[XPRE];
#pragma unroll
  for (int j = 0; j < XPRE; ++j)
    if (wave + 4 * j < nsb_x) xpre[j] = *(const float4 *)(x + (wave + 4 * j) * 256 + lane * 4);
  /* the other workgroups need the set of experts only, which mostly needs no exponential */
  const int item = blockIdx.y; /* < topk */
  unsigned long long set[MAXV];
  int e;
  if (topk_set_fast<MAXV>(logits, E, topk, set)) {
    e = nth_of_set<MAXV>(set, item);
  } else {
    route_token_regs<MAXV>(logits, 0, E, topk, renorm, myi, myw);
    const int rank = rank_by_expert(myi, topk);
    const unsigned long long owner = __ballot(lane < topk && rank == item);
    e = __shfl(myi, __ffsll((long long)owner) - 1, 64);
  }
  e = __builtin_amdgcn_readfirstlane(e);
  const WView wg = views[e], wu = views[E + e];
  const int K = wg.K;
  const XLds l = xlds_carve(xmoe_lds, TC, K);
  /* One tile of 32 columns a workgroup, a wavefront for each of (gate, up) x (first, second half of K):
   * with one wavefront per SIMD a super-block's eight matrix steps wait for each other, so half the
   * super-blocks per wavefront halve the stream's time. The chain of fp32 sums keeps the reference's
   * order: the second half's wavefront leaves its super-blocks' terms in LDS, and the first half's adds
   * them to its own after the barrier, one super-block after the other. */
  const int col0 = blockIdx.x * 32; /* < I: the grid has as many columns (and the one that routes) */
  const int first = wave >> 1, half = wave & 1; /* 0: gate, 1: up; which half of K */
  const int i32 = lane & 31, g = lane >> 5;
  const int nsb = K >> 8, n0 = (nsb + 1) >> 1; /* the first half's super-blocks */
  const int sb0 = half ? n0 : 0, cnt = half ? nsb - n0 : n0;
  float *terms = (float *)(xmoe_lds + xlds_bytes(TC, K)); /* [gate, up][super-block of the second half][4 terms][32 columns] */
  float *xch = terms + 2 * one_token_terms(K);            /* [32 columns] the gate values */
  auto stage = [&]() {
    /* rows 1 .. 7 of the matrix operand keep what the LDS held: a row of the product depends on
     * its own activations only, and those rows are not stored */
#pragma unroll
    for (int j = 0; j < XPRE; ++j) {
      const int b = wave + 4 * j;
      if (b < nsb) /* uniform per wavefront */
        hipq_quantize_q8_K_values<Q8K_ROWMMA>(xpre[j], 0, b, b, nsb, 0, l.q, l.dA, nullptr, nullptr,
                                              (uint16_t *)l.amin, nullptr, nullptr, TC);
    }
    for (int b = wave + 4 * XPRE; b < nsb; b += 4) { /* longer rows: the rest as it comes */
      const float4 xv = *(const float4 *)(x + b * 256 + lane * 4);
      hipq_quantize_q8_K_values<Q8K_ROWMMA>(xv, 0, b, b, nsb, 0, l.q, l.dA, nullptr, nullptr, (uint16_t *)l.amin,
                                            nullptr, nullptr, TC);
    }
    __syncthreads();
  };
  /* the tile (nibbles and headers of its super-blocks) as a buffer descriptor in scalar registers */
  const uint8_t *qs = first ? wu.qs : wg.qs;
  const xrsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
    (void *)(qs + (size_t)(col0 >> 5) * (size_t)(nsb * hipq::EXPERT_TILE_BYTES)), 0, nsb * hipq::EXPERT_TILE_BYTES,
    0x00020000);
  auto load = [&](XRegs &r, int sb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) /* non-temporal: every load instruction covers whole cache lines */
      r.q[i] = __builtin_bit_cast(
        mv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, lane * 16, sb * hipq::EXPERT_TILE_BYTES + i * 1024, 2));
    r.hd = __builtin_bit_cast(
      mv4i, __builtin_amdgcn_raw_buffer_load_b128(rq, 4096 + i32 * 16, sb * hipq::EXPERT_TILE_BYTES, 2));
  };
  /* Every step issues its loads whether or not a super-block is left: past the wavefront's last one the loads
   * name the descriptor's end and return zeros without touching memory. Behind a condition the waits could
   * not count them, and every super-block's arithmetic waited for the loads just issued for the next. */
  XRegs buf[2];
  load(buf[0], cnt > 0 ? sb0 : nsb);
  stage(); /* the row of x is quantized while the first weights are on their way */
  float acc = 0.f, accm = 0.f;
  for (int u0 = 0; u0 < cnt; u0 += 2) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int u = u0 + k;
      if (u < cnt) { /* uniform per wavefront */
        load(buf[(k + 1) & 1], u + 1 < cnt ? sb0 + u + 1 : nsb);
        float fi[NREG], si[NREG], fm[NREG], sm[NREG];
        xr_sb_terms<TC, NREG>(buf[k], l, K, sb0 + u, i32, g, fi, si, fm, sm);
        if (half == 0) {
          acc = fmaf(fi[0], si[0], acc);
          accm = fmaf(fm[0], sm[0], accm);
        } else if (lane < 32) {
          float *t = terms + (size_t)((first * one_token_terms(K) / 128 + u) * 4) * 32 + lane;
          t[0] = fi[0], t[32] = si[0], t[64] = fm[0], t[96] = sm[0];
        }
      }
    }
  }
  __syncthreads();
  float out = 0.f;
  if (half == 0) {
    for (int u = 0; u < nsb - n0; ++u) {
      const float *t = terms + (size_t)((first * one_token_terms(K) / 128 + u) * 4) * 32 + i32;
      acc = fmaf(t[0], t[32], acc);
      accm = fmaf(t[64], t[96], accm);
    }
    out = acc - accm;
    if (first == 0 && lane < 32) xch[lane] = out;
  }
  __syncthreads();
  if (first == 1 && half == 0 && lane < 32) {
    const int col = col0 + lane;
    if (col < I) h[(size_t)item * I + col] = moe_act(ep, e, I, col, xch[lane], out);
  }
}

/* QH: the rows of h come as fp32 (hf) and the workgroup quantizes those of its item
 * itself while its first weights are on their way, with the quantizer kernel's
 * arithmetic. Every column workgroup of an item repeats that, which pays with few
 * items (a decode step: one launch less), not with many. */
template <int TC, bool QH>
__global__ __launch_bounds__(256, TC <= 8 ? 4 : TC <= 16 ? 2 : 1) void down_mma_kernel(
  const WView *__restrict__ views, int E_, QView hq, const float *__restrict__ hf,
  const int *__restrict__ offsets, const int *__restrict__ items, const int *__restrict__ slot_pair,
  const float *__restrict__ wgt, int H, float *__restrict__ contrib, int ct, hipq::MoeEpi ep) {
  constexpr int NREG = TC / 2;
  extern __shared__ __attribute__((aligned(16))) unsigned char xmoe_lds[];
  const int item = blockIdx.y;
  if (item >= items[0]) return;
  const int e = items[2 + 2 * item], s0 = items[3 + 2 * item];
  const int end = min(s0 + TC, offsets[e + 1]);
  const WView wd = views[2 * E_ + e];
  const int K = wd.K;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const XLds l = xlds_carve(xmoe_lds, TC, K);
  const int col0 = (blockIdx.x * 4 + wave) * 32 * ct;
  const int ntile = min(ct, (H - col0 + 31) / 32);
  auto stage = [&]() {
    if (QH) {
      /* rows past the item's end stay as they are: a row of the matrix product
       * depends on its own activations only, and those rows are not stored */
      const int nsb = K >> 8, units = (end - s0) * nsb;
      for (int u0 = wave; u0 < units; u0 += 16) { /* uniform per wavefront; four loads, then four quantizations */
        float4 xv[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int u = min(u0 + 4 * k, units - 1), r = u / nsb, b = u - r * nsb;
          xv[k] = *(const float4 *)(hf + (size_t)(s0 + r) * K + b * 256 + lane * 4);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int u = u0 + 4 * k;
          if (u < units) {
            const int r = u / nsb, b = u - r * nsb;
            hipq_quantize_q8_K_values<Q8K_ROWMMA>(xv[k], 0, b, b, nsb, 0, l.q + (size_t)r * (K + 16), l.dA + r,
                                                  nullptr, nullptr, (uint16_t *)(l.amin + (size_t)r * nsb * 32),
                                                  nullptr, nullptr, TC);
          }
        }
      }
      __syncthreads();
      return;
    }
    if (threadIdx.x < TC) l.rows[threadIdx.x] = min(s0 + (int)threadIdx.x, end - 1); /* hq rows are slots */
    __syncthreads();
    stage_rows<TC>(l, hq, end - s0);
    __syncthreads();
  };
  if (ntile <= 0) {
    stage();
    return;
  }
  /* the routing weights of this lane's rows are asked for now: two dependent reads that would
   * otherwise stand between the last super-block and the store */
  float wrow[NREG];
#pragma unroll
  for (int r = 0; r < NREG; ++r) {
    const int tok = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
    wrow[r] = wgt[slot_pair[min(s0 + tok, end - 1)]];
  }
  xr_run<TC, NREG, XPD>(
    ntile, l, K,
    [&](int t, WView &w, int &c0) {
      w = wd;
      c0 = col0 + 32 * t;
    },
    [&](int t, const float(&out)[NREG]) {
      const int col = col0 + 32 * t + (lane & 31);
#pragma unroll
      for (int r = 0; r < NREG; ++r) {
        const int tok = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (col < H && s0 + tok < end) contrib[(size_t)(s0 + tok) * H + col] = moe_out(ep, e, H, col, out[r], wrow[r]);
      }
    },
    stage);
}

/* ---- The block without a pair sort ------------------------------------------------------
 * For chunks of a few dozen tokens the sort is a launch of its own (4-5 us of a block of 80) and
 * puts three dependent reads (item, offsets, pairs) in front of every workgroup's first weight
 * load. Here a workgroup is given (expert, chunk of 16 of its pairs) by its block id and finds the
 * pairs itself in the routing's idx[P] (a few KB: every thread compares its share, ranks by pair
 * number come from a prefix sum over the workgroup). Rows of h and of the contributions are
 * numbered by pair, and the routing writes each token's pairs in ascending expert id for the
 * combine. An expert with up to 8 pairs runs the 8-row form of the matrix step, one with 9 to 16
 * the 16-row form, so either is ONE workgroup per column block: its weights cross HBM once and the
 * number of streaming workgroups is the number of active experts whatever the routing (with 128
 * experts and 768 intermediate columns exactly three on every CU). Experts with more than 16 pairs
 * continue in the next row of the grid (blockIdx.y / E); rows whose chunk is empty leave after the
 * scan. */
constexpr int SELF_TC = 16;     /* pairs per chunk */
constexpr int SELF_HEAD = 128;  /* bytes of LDS in front of the rows: pairs[16], tokens[16] */

/* The scan of the routing's output in two parts, so that a workgroup can ask for other things
 * between them: the loads of idx (up to four pairs per thread in registers; longer lists are read
 * in the second part), then the counting. */
struct SelfAsk {
  int v[4];
};

__device__ __forceinline__ SelfAsk self_scan_ask(const int32_t *__restrict__ idx, int P) {
  const int t = threadIdx.x;
  const int pp = (P + 255) >> 8; /* pairs per thread, consecutive: thread order is pair order */
  SelfAsk a;
#pragma unroll
  for (int u = 0; u < 4; ++u) a.v[u] = idx[min(t * pp + min(u, pp - 1), P - 1)];
  return a;
}

__device__ __forceinline__ int self_scan(const SelfAsk &a, const int32_t *__restrict__ idx, int P, int topk, int e,
                                         int chunk, int *pairs, int *rows) {
  __shared__ int wtot[4];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int pp = (P + 255) >> 8;
  int m = 0;
  uint32_t mask = 0;
  if (pp <= 4) { /* uniform */
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < pp && t * pp + u < P && a.v[u] == e) mask |= 1u << u, ++m;
  } else {
    for (int u = 0; u < pp; ++u) {
      const int i = t * pp + u;
      if (i < P && idx[i] == e) mask |= 1u << u, ++m;
    }
  }
  const int inc = hipq_wave_prefix_sum_i(m); /* inclusive, over the lanes */
  if (lane == 63) wtot[wave] = inc;
  __syncthreads();
  int base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    base += w < wave ? wtot[w] : 0;
    total += wtot[w];
  }
  int r = base + inc - m - chunk * SELF_TC;
  for (int u = 0; u < pp; ++u)
    if (mask >> u & 1) {
      if (r >= 0 && r < SELF_TC) {
        pairs[r] = t * pp + u;
        rows[r] = (t * pp + u) / topk;
      }
      ++r;
    }
  __syncthreads();
  return total;
}

/* Load instructions that touch every cache line of a wavefront's first NT super-blocks of column
 * tile `tile` (a lane per 128 bytes, one instruction a super-block), so that the lines are on their
 * way to the caches while the workgroup finds its pairs and stages its rows. The values come back in
 * NT registers, which self_touched() takes behind the staging's barrier. */
/* One super-block: touching two or three made the block 1-4 us slower (the lines do not stay in
 * the L2 until they are used). */
constexpr int SELF_TOUCH = 1;
template <int NT> struct SelfTouch {
  int v[NT];
};
template <int NT> __device__ __forceinline__ void self_touch(SelfTouch<NT> &t, const WView &w, int tile) {
  const int nsb = w.K >> 8, lane = threadIdx.x & 63;
  const xrsrc_t rq =
    __builtin_amdgcn_make_buffer_rsrc((void *)(w.qs + (size_t)tile * (size_t)(nsb * hipq::EXPERT_TILE_BYTES)), 0,
                                      min(NT, nsb) * hipq::EXPERT_TILE_BYTES, 0x00020000);
#pragma unroll
  for (int i = 0; i < NT; ++i) /* lanes past a super-block's end, and super-blocks past the tile's, read nothing */
    t.v[i] = __builtin_amdgcn_raw_buffer_load_b32(rq, lane < hipq::EXPERT_TILE_BYTES / 128 ? lane * 128 : 0x7fffff00,
                                                  i * hipq::EXPERT_TILE_BYTES, 0);
}
template <int NT> __device__ __forceinline__ void self_touched(const SelfTouch<NT> &t) {
#pragma unroll
  for (int i = 0; i < NT; ++i) asm volatile("" ::"v"(t.v[i]));
}

template <int TC>
__device__ __forceinline__ void gate_up_self_pass(unsigned char *lds, int n, int e, const WView &wg, const WView &wu,
                                                  const QView &xq, int I, float *__restrict__ h,
                                                  const hipq::MoeEpi &ep, const SelfTouch<SELF_TOUCH> &touched) {
  constexpr int NREG = TC / 2;
  const int K = wg.K;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  XLds l = xlds_carve(lds + SELF_HEAD, TC, K);
  l.pairs = (int *)lds;
  l.rows = l.pairs + SELF_TC;
  const int col0 = (blockIdx.x * 4 + wave) * 32;
  const uint64_t dqs = (uint64_t)wu.qs - (uint64_t)wg.qs;
  auto stage = [&]() {
    stage_rows<TC>(l, xq, n);
    __syncthreads();
    self_touched(touched);
  };
  if (col0 >= I) { /* uniform per wavefront; it still takes part in the barrier */
    stage();
    return;
  }
  float gate[NREG], up[NREG];
  xr_run<TC, NREG, XPD>(
    2, l, K,
    [&](int t, WView &w, int &c0) {
      const uint64_t isup = (uint64_t)0 - (uint64_t)(t & 1);
      w.qs = (const uint8_t *)((uint64_t)wg.qs + (isup & dqs));
      w.hdr = nullptr; /* the headers follow the nibbles */
      w.N = wg.N;
      w.K = wg.K;
      c0 = col0;
    },
    [&](int t, const float(&out)[NREG]) {
      if (t == 0) {
#pragma unroll
        for (int r = 0; r < NREG; ++r) gate[r] = out[r];
      } else {
#pragma unroll
        for (int r = 0; r < NREG; ++r) up[r] = out[r];
      }
    },
    stage);
  const int col = col0 + (lane & 31);
#pragma unroll
  for (int r = 0; r < NREG; ++r) {
    const int tok = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
    if (col < I && tok < n) h[(size_t)l.pairs[tok] * I + col] = moe_act(ep, e, I, col, gate[r], up[r]);
  }
}

__global__ __launch_bounds__(256, 4) void gate_up_self_kernel(const WView *__restrict__ views, int E_, QView xq,
                                                              const int32_t *__restrict__ idx, int P, int topk, int I,
                                                              float *__restrict__ h, hipq::MoeEpi ep) {
  extern __shared__ __attribute__((aligned(16))) unsigned char xmoe_lds[];
  const int e = blockIdx.y % E_, chunk = blockIdx.y / E_;
  const SelfAsk ask = self_scan_ask(idx, P);
  const WView wg = views[e], wu = views[E_ + e];
  /* a workgroup of the first chunk row has work unless nobody chose its expert: its first
   * weights start towards the L2 before it knows its pairs */
  const int col0 = (blockIdx.x * 4 + (int)(threadIdx.x >> 6)) * 32;
  SelfTouch<SELF_TOUCH> touched = {};
  if (chunk == 0 && col0 < I) self_touch(touched, wg, __builtin_amdgcn_readfirstlane(col0 >> 5));
  int *pairs = (int *)xmoe_lds;
  const int total = self_scan(ask, idx, P, topk, e, chunk, pairs, pairs + SELF_TC);
  const int n = min(SELF_TC, total - chunk * SELF_TC);
  if (n <= 0) return; /* uniform per workgroup */
  if (n <= 8)
    gate_up_self_pass<8>(xmoe_lds, n, e, wg, wu, xq, I, h, ep, touched);
  else {
    /* a workgroup of the 16-row form has the longest way (its steps carry twice the rows): its wavefronts go
     * first on their SIMDs, so that the launch does not end on them (64-token blocks whose routing has
     * experts with nine pairs and more: 81.7 -> 78.4 and 77.0 -> 74.9 us, three runs each) */
    __builtin_amdgcn_s_setprio(2);
    gate_up_self_pass<16>(xmoe_lds, n, e, wg, wu, xq, I, h, ep, touched);
  }
}

/* The rows of h come as fp32 and the workgroup quantizes those of its chunk itself while its first
 * weights are on their way (the QH form of down_mma_kernel). */
template <int TC>
__device__ __forceinline__ void down_self_pass(unsigned char *lds, int n, int e, const WView &wd,
                                               const float *__restrict__ hf, const float *__restrict__ wgt,
                                               int H, float *__restrict__ contrib, const hipq::MoeEpi &ep,
                                               const SelfTouch<SELF_TOUCH> &touched) {
  constexpr int NREG = TC / 2, CT = 2;
  const int K = wd.K;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  XLds l = xlds_carve(lds + SELF_HEAD, TC, K);
  l.pairs = (int *)lds;
  l.rows = l.pairs + SELF_TC;
  const int col0 = (blockIdx.x * 4 + wave) * 32 * CT;
  const int ntile = min(CT, (H - col0 + 31) / 32);
  auto stage = [&]() {
    /* rows past the chunk's end stay as they are: a row of the matrix product depends on its own
     * activations only, and those rows are not stored */
    const int nsb = K >> 8, units = n * nsb;
    /* a wavefront's (row, super-block) units four at a time: the four loads first, then the four
     * quantizations (one after the other, a unit's load is a round trip of its own: 4-6 us of this
     * kernel's start with three rows of three super-blocks) */
    for (int u0 = wave; u0 < units; u0 += 16) { /* uniform per wavefront */
      float4 xv[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int u = min(u0 + 4 * k, units - 1), r = u / nsb, b = u - r * nsb;
        xv[k] = *(const float4 *)(hf + (size_t)l.pairs[r] * K + b * 256 + lane * 4);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int u = u0 + 4 * k;
        if (u < units) {
          const int r = u / nsb, b = u - r * nsb;
          hipq_quantize_q8_K_values<Q8K_ROWMMA>(xv[k], 0, b, b, nsb, 0, l.q + (size_t)r * (K + 16), l.dA + r, nullptr,
                                                nullptr, (uint16_t *)(l.amin + (size_t)r * nsb * 32), nullptr,
                                                nullptr, TC);
        }
      }
    }
    __syncthreads();
    self_touched(touched);
  };
  if (ntile <= 0) {
    stage();
    return;
  }
  xr_run<TC, NREG, XPD>(
    ntile, l, K,
    [&](int t, WView &w, int &c0) {
      w = wd;
      c0 = col0 + 32 * t;
    },
    [&](int t, const float(&out)[NREG]) {
      const int col = col0 + 32 * t + (lane & 31);
#pragma unroll
      for (int r = 0; r < NREG; ++r) {
        const int tok = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (col < H && tok < n) {
          const int pair = l.pairs[tok];
          contrib[(size_t)pair * H + col] = moe_out(ep, e, H, col, out[r], wgt[pair]);
        }
      }
    },
    stage);
}

__global__ __launch_bounds__(256, 4) void down_self_kernel(const WView *__restrict__ views, int E_,
                                                           const float *__restrict__ hf,
                                                           const int32_t *__restrict__ idx, int P, int topk,
                                                           const float *__restrict__ wgt, int H,
                                                           float *__restrict__ contrib, hipq::MoeEpi ep) {
  extern __shared__ __attribute__((aligned(16))) unsigned char xmoe_lds[];
  const int e = blockIdx.y % E_, chunk = blockIdx.y / E_;
  const SelfAsk ask = self_scan_ask(idx, P);
  const WView wd = views[2 * E_ + e];
  const int col0 = (blockIdx.x * 4 + (int)(threadIdx.x >> 6)) * 64; /* two column tiles per wavefront */
  SelfTouch<SELF_TOUCH> touched = {};
  if (chunk == 0 && col0 < H) self_touch(touched, wd, __builtin_amdgcn_readfirstlane(col0 >> 5));
  int *pairs = (int *)xmoe_lds;
  const int total = self_scan(ask, idx, P, topk, e, chunk, pairs, pairs + SELF_TC);
  const int n = min(SELF_TC, total - chunk * SELF_TC);
  if (n <= 0) return; /* uniform per workgroup */
  if (n <= 8)
    down_self_pass<8>(xmoe_lds, n, e, wd, hf, wgt, H, contrib, ep, touched);
  else {
    __builtin_amdgcn_s_setprio(2); /* as in gate_up_self_kernel */
    down_self_pass<16>(xmoe_lds, n, e, wd, hf, wgt, H, contrib, ep, touched);
  }
}

/* y[t][c] = sum of the token's contributions, ascending expert id */
__global__ __launch_bounds__(256) void combine_kernel(const int *__restrict__ tok_slots, int topk,
                                                      int H, const float *__restrict__ contrib,
                                                      float *__restrict__ y) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= H) return;
  float acc = 0.f;
  for (int k0 = 0; k0 < topk; k0 += 8) { /* eight loads in flight, added in order */
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
      v[k] = k0 + k < topk ? contrib[(size_t)tok_slots[t * topk + k0 + k] * H + c] : 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (k0 + k < topk) acc = acc + v[k];
  }
  y[(size_t)t * H + c] = acc;
}

/* Lanes per weight row, chunk size and weight rows per wavefront for rows of K
 * weights: expert matrices are short (K = 768 .. 4096), so the lanes of a
 * wavefront are split over 4, 2 or 1 rows such that (nearly) all of them hold a
 * unit, and more rows per wavefront amortise the activation loads. Q6_K has eight
 * fp32 chains per output, which bounds the rows per wavefront. */
constexpr int CPW = 4; /* column groups per wavefront */

template <int DT, int T, int KC, int G>
void launch_gate_up(const hipq_moe_desc &d, const hipq::MoeEpi &ep, const WView *views, const QAct &xq,
                    const MoeBufs &b, hipStream_t s) {
  const size_t lds = 4 * GemvLds<DT, RTOK, G, false>::DWORDS * sizeof(uint32_t);
  if (d.hidden > KC) {
    const dim3 grid((d.intermediate + 7) / 8, d.experts);
    const size_t lds_long = 4 * GemvLds<DT, RTOK, 2, false>::DWORDS * sizeof(uint32_t);
    hipq::launch_kernel("gate_up_long_kernel<DT>", (gate_up_long_kernel<DT>), grid, dim3(256), lds_long, s, views, d.experts,
                       qview(xq), b.offsets, b.slot_pair, d.topk, d.intermediate, b.h, ep);
    return;
  }
  const dim3 grid((d.intermediate + 4 * G * CPW - 1) / (4 * G * CPW), d.experts);
  hipq::launch_kernel("gate_up_kernel<DT, T, KC, G, CPW>", (gate_up_kernel<DT, T, KC, G, CPW>), grid, dim3(256), lds, s, views, d.experts,
                     qview(xq), b.offsets, b.slot_pair, d.topk, d.intermediate, b.h, ep);
}
template <int DT, int T, int KC, int G>
void launch_down(const hipq_moe_desc &d, const hipq::MoeEpi &ep, const WView *views, const QAct &hq,
                 const MoeBufs &b, hipStream_t s) {
  const size_t lds = 4 * GemvLds<DT, RTOK, G, false>::DWORDS * sizeof(uint32_t);
  if (d.intermediate > KC) {
    const dim3 grid((d.hidden + 7) / 8, d.experts);
    const size_t lds_long = 4 * GemvLds<DT, RTOK, 2, false>::DWORDS * sizeof(uint32_t);
    hipq::launch_kernel("down_long_kernel<DT>", (down_long_kernel<DT>), grid, dim3(256), lds_long, s, views, d.experts,
                       qview(hq), b.offsets, b.slot_pair, b.wgt, d.hidden, b.contrib, ep);
    return;
  }
  const dim3 grid((d.hidden + 4 * G * CPW - 1) / (4 * G * CPW), d.experts);
  hipq::launch_kernel("down_kernel<DT, T, KC, G, CPW>", (down_kernel<DT, T, KC, G, CPW>), grid, dim3(256), lds, s, views, d.experts,
                     qview(hq), b.offsets, b.slot_pair, b.wgt, d.hidden, b.contrib, ep);
}

/* calls f.template operator()<T, KC, G>() for the shape class of K */
template <int DT, typename F> void for_row_length(int64_t K, F f) {
  if constexpr (DT == HIPQ_Q4_K) {
    if (K <= 1024) f.template operator()<16, 1024, 8>();
    else if (K <= 2048) f.template operator()<32, 2048, 4>();
    else f.template operator()<64, 4096, 4>();
  } else if constexpr (DT == HIPQ_Q4_0) {
    if (K <= 1024) f.template operator()<32, 1024, 2>();
    else if (K <= 2048) f.template operator()<64, 2048, 2>();
    else f.template operator()<64, 4096, 2>();
  } else {
    if (K <= 2048) f.template operator()<32, 2048, 2>();
    else f.template operator()<64, 4096, 2>();
  }
}

template <int DT> struct GateUpLauncher {
  const hipq_moe_desc &d;
  const hipq::MoeEpi &ep;
  const WView *views;
  const QAct &xq;
  const MoeBufs &b;
  hipStream_t s;
  template <int T, int KC, int G> void operator()() const { launch_gate_up<DT, T, KC, G>(d, ep, views, xq, b, s); }
};
template <int DT> struct DownLauncher {
  const hipq_moe_desc &d;
  const hipq::MoeEpi &ep;
  const WView *views;
  const QAct &hq;
  const MoeBufs &b;
  hipStream_t s;
  template <int T, int KC, int G> void operator()() const { launch_down<DT, T, KC, G>(d, ep, views, hq, b, s); }
};

constexpr size_t XLDS_MAX = 160 * 1024; /* LDS of a CU */

/* Few work items: halve the gate/up stream of a wavefront and give the down product
 * one column tile per wavefront instead of two (its rows are short), so that more
 * wavefronts share the weights' bytes. */
bool mma_few(const hipq_moe_desc &d, int TC) {
  const int64_t P = (int64_t)d.tokens * d.topk;
  const int64_t max_items = (P < d.experts ? P : d.experts) + P / TC;
  return max_items * ((d.intermediate + 127) / 128) * 4 <= 2048;
}
/* The block without a pair sort: the regime of 8-token chunks (a mean expert has at most four
 * pairs), more tokens than the one-launch routing and sort of a decode step takes, an idx[] that
 * a workgroup scans in one go, and rows short enough that four workgroups of the 16-row form fit
 * a CU's LDS. */
bool mma_self(const hipq_moe_desc &d, int TC) {
  const int64_t P = (int64_t)d.tokens * d.topk;
  const int kmax = d.hidden > d.intermediate ? d.hidden : d.intermediate;
  return TC == 8 && !mma_few(d, TC) && d.tokens > 16 && P <= 1024 && d.topk <= 64 &&
         4 * (SELF_HEAD + xlds_bytes(SELF_TC, kmax)) <= XLDS_MAX;
}
int launch_self_mma(const hipq::MoeArgs *a, const MoeBufs &b, const WView *views, const QAct &xq, hipStream_t s) {
  const hipq_moe_desc &d = a->desc;
  const int P = d.tokens * d.topk;
  const unsigned gy = (unsigned)(((d.tokens + SELF_TC - 1) / SELF_TC) * d.experts); /* an expert has at most T pairs */
  const size_t lds_g = SELF_HEAD + xlds_bytes(SELF_TC, d.hidden), lds_d = SELF_HEAD + xlds_bytes(SELF_TC, d.intermediate);
  hipq::launch_kernel("gate_up_self_kernel", gate_up_self_kernel, dim3((d.intermediate + 127) / 128, gy), dim3(256), lds_g, s,
                      views, d.experts, qview(xq), b.idx_used, P, d.topk, d.intermediate, b.h, a->epi);
  HIPQ_HIP(hipGetLastError());
  hipq::launch_kernel("down_self_kernel", down_self_kernel, dim3((d.hidden + 255) / 256, gy), dim3(256), lds_d, s, views,
                      d.experts, (const float *)b.h, b.idx_used, P, d.topk, (const float *)b.wgt, d.hidden, b.contrib,
                      a->epi);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

template <int TC>
int launch_grouped_mma(const hipq::MoeArgs *a, const MoeBufs &b, const WView *views, const QAct &xq,
                       const QAct &hq, hipStream_t s, bool gate_up_done = false) {
  const hipq_moe_desc &d = a->desc;
  const int64_t P = (int64_t)d.tokens * d.topk;
  /* an upper bound of the work items: one per active expert and one per full chunk */
  const int max_items = (int)((P < d.experts ? P : d.experts) + P / TC);
  const bool few = mma_few(d, TC);
  const size_t lds_g = xlds_bytes(TC, d.hidden) + (few ? TC * 256 : 0);
  const size_t lds_d = xlds_bytes(TC, d.intermediate);
  const void *kg = few ? (const void *)gate_up_mma_kernel<TC, true> : (const void *)gate_up_mma_kernel<TC, false>;
  if (lds_g > 64 * 1024) /* beyond the default limit of a launch */
    HIPQ_HIP(hipFuncSetAttribute(kg, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_g));
  if (gate_up_done) {
    /* h is there: the routing launch formed it (gate_up_one_token_kernel) */
  } else if (few)
    hipq::launch_kernel("gate_up_mma_kernel<TC, true>", (gate_up_mma_kernel<TC, true>), dim3((d.intermediate + 63) / 64, max_items), dim3(256), lds_g,
                       s, views, d.experts, qview(xq), b.offsets, b.items, b.slot_pair, d.topk, d.intermediate,
                       b.h, a->epi);
  else
    hipq::launch_kernel("gate_up_mma_kernel<TC, false>", (gate_up_mma_kernel<TC, false>), dim3((d.intermediate + 127) / 128, max_items), dim3(256),
                       lds_g, s, views, d.experts, qview(xq), b.offsets, b.items, b.slot_pair, d.topk,
                       d.intermediate, b.h, a->epi);
  HIPQ_HIP(hipGetLastError());
  /* the down kernel quantizes its item's rows of h itself (QH): one launch less. With many items
   * every column workgroup of an item repeats the rows, which costs less than the launch did
   * (92.6 -> 90.3 us at 64 tokens). The launch-a-quantizer form stays for rows too long to be
   * quantized inside a workgroup's start-up. */
  const bool qh = true;
  if (!qh) {
    int rc = hipq::launch_quantize_q8_K_rowmma(b.h, P, d.intermediate, d.intermediate, &hq, s);
    if (rc) return rc;
  }
  const void *kd = qh ? (const void *)down_mma_kernel<TC, true> : (const void *)down_mma_kernel<TC, false>;
  if (lds_d > 64 * 1024)
    HIPQ_HIP(hipFuncSetAttribute(kd, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_d));
  const int ct = few ? 1 : 2;
  const dim3 gd((d.hidden + 128 * ct - 1) / (128 * ct), max_items);
  if (qh)
    hipq::launch_kernel("down_mma_kernel<TC, true>", (down_mma_kernel<TC, true>), gd, dim3(256), lds_d, s, views, d.experts, qview(hq), b.h,
                       b.offsets, b.items, b.slot_pair, b.wgt, d.hidden, b.contrib, ct, a->epi);
  else
    hipq::launch_kernel("down_mma_kernel<TC, false>", (down_mma_kernel<TC, false>), gd, dim3(256), lds_d, s, views, d.experts, qview(hq), b.h,
                       b.offsets, b.items, b.slot_pair, b.wgt, d.hidden, b.contrib, ct, a->epi);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

/* Token chunk of the matrix-core expert kernels for P pairs over E experts: the
 * smallest of 8, 16, 32 that holds twice the mean tokens per expert (an expert with
 * more becomes several work items), reduced until the activation rows fit the LDS. */
int mma_chunk(const hipq_moe_desc &d, int64_t P, int E) {
  const int64_t mean2 = (2 * P + E - 1) / E;
  int tc = mean2 <= 8 ? 8 : mean2 <= 16 ? 16 : 32;
  const int kmax = d.hidden > d.intermediate ? d.hidden : d.intermediate;
  while (tc > 8 && xlds_bytes(tc, kmax) + tc * 256 > XLDS_MAX) tc >>= 1; /* + the paired form's exchange area */
  return tc;
}
bool use_mma(const hipq_moe_desc &d, int dt) {
  const int kmax = d.hidden > d.intermediate ? d.hidden : d.intermediate;
  return dt == HIPQ_Q4_K && xlds_bytes(8, kmax) + 8 * 256 <= XLDS_MAX;
}

template <int DT>
int launch_grouped(const hipq::MoeArgs *a, const MoeBufs &b, const WView *views, const QAct &xq,
                   const QAct &hq, hipStream_t s) {
  const hipq_moe_desc &d = a->desc;
  const int64_t P = (int64_t)d.tokens * d.topk;
  int rc;
  for_row_length<DT>(d.hidden, GateUpLauncher<DT>{d, a->epi, views, xq, b, s});
  HIPQ_HIP(hipGetLastError());
  if (DT == HIPQ_Q4_0)
    rc = hipq::launch_quantize_q8_0(b.h, P, d.intermediate, d.intermediate, &hq, nullptr, s);
  else
    rc = hipq::launch_quantize_q8_K(b.h, P, d.intermediate, d.intermediate, 0, &hq, nullptr, s);
  if (rc) return rc;
  for_row_length<DT>(d.intermediate, DownLauncher<DT>{d, a->epi, views, hq, b, s});
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace

namespace hipq {

bool moe_wants_tiles(const hipq_moe_desc *d, int dtype) { return use_mma(*d, dtype); }

size_t moe_workspace_bytes(const hipq_moe_desc *d) {
  /* sized for the larger (Q8_K) activation form */
  return carve(*d, 1, nullptr, nullptr);
}

int launch_moe(const MoeArgs *a, void *workspace, size_t workspace_bytes, const WView *views,
               hipStream_t s) {
  const hipq_moe_desc &d = a->desc;
  const int dt = a->gate[0]->dtype;
  const int is_k = dt != HIPQ_Q4_0;
  const int blk = is_k ? 256 : 32;
  if (d.hidden % blk || d.intermediate % blk)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "hidden %d and intermediate %d must be multiples of %d",
                d.hidden, d.intermediate, blk);
  MoeBufs b;
  const size_t need = carve(d, is_k, (uint8_t *)workspace, &b);
  if (need > workspace_bytes) return fail(HIPQ_ERR_RUNTIME, "MoE workspace too small");
  const int T = d.tokens, E = d.experts, P = T * d.topk;

  const float *logits = a->router_logits;
  if (!logits) {
    /* the rows of x of a workgroup's tokens go to LDS: four tokens, or as many as there are or fit 64 KB with the partial sums */
    int tb_n = d.hidden > 0 ? (int)std::min<int64_t>(std::min(ROUTER_TB, T), 15000 / d.hidden) : 0;
    tb_n = tb_n >= 4 ? 4 : tb_n >= 2 ? 2 : tb_n;
    if ((E & 3) || (d.hidden & 3) || tb_n < 1 || (((uintptr_t)a->router_weight | (uintptr_t)a->x) & 15)) {
      hipq::launch_kernel("router_logits_scalar_kernel", router_logits_scalar_kernel, dim3(T), dim3(256), 0, s, a->x,
                          a->router_weight, d.hidden, E, a->router_bias, b.logits);
    } else {
      const dim3 grid((E / 4 + 3) / 4, (T + tb_n - 1) / tb_n);
      const size_t lds = router_lds_bytes(tb_n, d.hidden);
      auto launch = [&](auto k, const char *name) {
        hipq::launch_kernel(name, k, grid, dim3(256), lds, s, a->x, a->router_weight, T, d.hidden, E, a->router_bias,
                            b.logits);
      };
      if (tb_n == 4) launch(router_logits_kernel<4>, "router_logits_kernel<4>");
      else if (tb_n == 2) launch(router_logits_kernel<2>, "router_logits_kernel<2>");
      else launch(router_logits_kernel<1>, "router_logits_kernel<1>");
    }
    HIPQ_HIP(hipGetLastError());
    logits = b.logits;
  }
  const bool mma = use_mma(d, dt);
  const int chunk = mma ? mma_chunk(d, P, E) : 0; /* tokens of an expert per work item of the matrix-core kernels */
  int32_t *idx = a->topk_idx ? a->topk_idx : b.idx;
  float *wgt = a->topk_w ? a->topk_w : b.wgt;
  b.wgt = wgt;
  b.idx_used = idx;
  const bool self = mma && mma_self(d, chunk); /* no pair sort: the expert kernels find their pairs in idx */
  /* the router is instantiated for 2, 4 and 16 logits per lane (E <= 128, 256, 1024):
   * a short kernel whose code is mostly fetched cold, so its length is its time.
   * For the matrix-core expert kernels the same launch quantizes x. */
  QAct xq = qact_carve(is_k, b.xq_mem, T, d.hidden);
  QAct hq = qact_carve(is_k, b.hq_mem, P, d.intermediate);
  const XQuant xqa = {a->x, (int64_t)T * (d.hidden / 256), d.hidden / 256, xq.q, xq.d, (uint16_t *)xq.bsum};
  if (mma && (((uintptr_t)a->x & 15) != 0))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "activation rows must be 16-byte aligned");
  /* one token on the matrix-core path: routing, the quantization of x and gate/up as one launch */
  const bool one_token = mma && T == 1 && chunk == 8 && mma_few(d, 8) && E <= 1024 && d.topk <= 64;
  if (one_token) {
    const size_t lds_g = xlds_bytes(8, d.hidden) + (2 * (size_t)one_token_terms(d.hidden) + 32) * sizeof(float);
    if (lds_g > 64 * 1024) {
      const void *k = E <= 128   ? (const void *)gate_up_one_token_kernel<2>
                      : E <= 256 ? (const void *)gate_up_one_token_kernel<4>
                                 : (const void *)gate_up_one_token_kernel<16>;
      HIPQ_HIP(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_g));
    }
    /* one block column more than the columns of h need: the routing's outputs are written there */
    const dim3 grid((unsigned)((d.intermediate + 31) / 32) + 1, (unsigned)d.topk);
    auto launch = [&](auto k, const char *name) {
      hipq::launch_kernel(name, k, grid, dim3(256), lds_g, s, logits, E, d.topk, d.renormalize, idx, wgt, b.offsets,
                          b.slot_pair, b.tok_slots, b.items, a->x, views, d.hidden, d.intermediate, b.h, a->epi);
    };
    if (E <= 128) launch(gate_up_one_token_kernel<2>, "gate_up_one_token_kernel<2>");
    else if (E <= 256) launch(gate_up_one_token_kernel<4>, "gate_up_one_token_kernel<4>");
    else launch(gate_up_one_token_kernel<16>, "gate_up_one_token_kernel<16>");
    HIPQ_HIP(hipGetLastError());
  } else if (T <= 16 && E <= 1024) {
    const unsigned qblocks = mma ? (unsigned)((xqa.n_sb + 15) / 16) : 0;
    auto launch = [&](auto fused, auto plain) {
      if (mma)
        hipq::launch_kernel("fused", fused, dim3(1 + qblocks), dim3(1024), 0, s, logits, T, E, d.topk, d.renormalize, idx,
                           wgt, b.offsets, b.slot_pair, b.tok_slots, chunk, b.items, xqa);
      else
        hipq::launch_kernel("plain", plain, dim3(1), dim3(1024), 0, s, logits, T, E, d.topk, d.renormalize, idx, wgt,
                           b.offsets, b.slot_pair, b.tok_slots, chunk, b.items);
    };
    if (E <= 128) launch(route_sort_quantize_kernel<2>, route_sort_kernel<2>);
    else if (E <= 256) launch(route_sort_quantize_kernel<4>, route_sort_kernel<4>);
    else launch(route_sort_quantize_kernel<16>, route_sort_kernel<16>);
    HIPQ_HIP(hipGetLastError());
  } else {
    const int rblocks = (T + 3) / 4;
    const unsigned qblocks = mma ? (unsigned)((xqa.n_sb + 3) / 4) : 0;
    auto launch = [&](auto fused, auto plain) {
      if (mma)
        hipq::launch_kernel("fused", fused, dim3(rblocks + qblocks), dim3(256), 0, s, logits, T, E, d.topk, d.renormalize,
                           idx, wgt, rblocks, xqa, self ? b.tok_slots : (int *)nullptr);
      else
        hipq::launch_kernel("plain", plain, dim3(rblocks), dim3(256), 0, s, logits, T, E, d.topk, d.renormalize, idx, wgt);
    };
    if (E <= 128) launch(route_quantize_kernel<2>, route_kernel<2>);
    else if (E <= 256) launch(route_quantize_kernel<4>, route_kernel<4>);
    else launch(route_quantize_kernel<16>, route_kernel<16>);
    HIPQ_HIP(hipGetLastError());
  }
  if ((T <= 16 && E <= 1024) || self || one_token) {
    /* routed and sorted above, or no sort needed */
  } else if (P <= 16384 && E <= 1024) {
    hipq::launch_kernel("sort_pairs_kernel", sort_pairs_kernel, dim3(1), dim3(1024), 0, s, idx, P, E, d.topk, b.offsets,
                       b.slot_pair, b.tok_slots, chunk, b.items);
  } else {
    hipq::launch_kernel("fill_int_kernel", fill_int_kernel, dim3((E + 255) / 256), dim3(256), 0, s, b.counts, E, 0);
    hipq::launch_kernel("count_kernel", count_kernel, dim3((P + 255) / 256), dim3(256), 0, s, idx, P, b.counts);
    hipq::launch_kernel("scan_kernel", scan_kernel, dim3(1), dim3(64), 0, s, b.counts, E, b.offsets, b.cursor, chunk, b.items);
    hipq::launch_kernel("scatter_kernel", scatter_kernel, dim3((P + 255) / 256), dim3(256), 0, s, idx, P, d.topk, b.offsets,
                       b.cursor, b.slot_pair, b.tok_slots);
  }
  HIPQ_HIP(hipGetLastError());

  int rc = mma    ? HIPQ_OK /* quantized with the routing */
           : is_k ? launch_quantize_q8_K(a->x, T, d.hidden, d.hidden, 0, &xq, nullptr, s)
                  : launch_quantize_q8_0(a->x, T, d.hidden, d.hidden, &xq, nullptr, s);
  if (rc) return rc;
  if (self) {
    rc = launch_self_mma(a, b, views, xq, s);
  } else if (mma) {
    const int tc = chunk;
    rc = tc == 8    ? launch_grouped_mma<8>(a, b, views, xq, hq, s, one_token)
         : tc == 16 ? launch_grouped_mma<16>(a, b, views, xq, hq, s)
                    : launch_grouped_mma<32>(a, b, views, xq, hq, s);
  } else if (dt == HIPQ_Q4_0)
    rc = launch_grouped<HIPQ_Q4_0>(a, b, views, xq, hq, s);
  else if (dt == HIPQ_Q4_K)
    rc = launch_grouped<HIPQ_Q4_K>(a, b, views, xq, hq, s);
  else
    rc = launch_grouped<HIPQ_Q6_K>(a, b, views, xq, hq, s);
  if (rc) return rc;
  hipq::launch_kernel("combine_kernel", combine_kernel, dim3((d.hidden + 255) / 256, T), dim3(256), 0, s, b.tok_slots,
                     d.topk, d.hidden, b.contrib, a->y);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
