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
 * on device data): router logits (optional) -> route -> count -> scan ->
 * scatter (pairs sorted by expert) -> quantize x -> grouped gate+up GEMV with
 * fused SwiGLU over (column tiles x experts) -> quantize h -> grouped down GEMV
 * scaled by the routing weight -> combine. Within an expert the weight rows are
 * streamed once per group of four tokens. Each single-row product is computed by
 * the same engine as the decode GEMV, so it carries the reference's bits.
 */
#include "gemv_device.h"

namespace {

constexpr int RTOK = 4; /* tokens sharing one pass over an expert's weight rows */

struct MoeBufs {
  float *logits;
  int32_t *idx;
  float *wgt;
  int *counts, *offsets, *cursor;
  int *slot_pair, *pair_slot;
  float *h;       /* [P][I] by slot */
  float *contrib; /* [P][H] by slot */
  void *xq_mem, *hq_mem;
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
  if (b) b->pair_slot = (int *)p;
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

/* logits[t][e] = sum_h x[t][h] * Wr[h][e] */
__global__ __launch_bounds__(256) void router_logits_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ wr, int H,
                                                            int E, float *__restrict__ logits) {
  const int t = blockIdx.x;
  const float *xt = x + (size_t)t * H;
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    float acc = 0.f;
    for (int h = 0; h < H; ++h) acc = fmaf(xt[h], wr[(size_t)h * E + e], acc);
    logits[(size_t)t * E + e] = acc;
  }
}

/* One wavefront per token: softmax, top-k, optional renormalisation. */
__global__ __launch_bounds__(256) void route_kernel(const float *__restrict__ logits, int T, int E,
                                                    int topk, int renorm,
                                                    int32_t *__restrict__ idx,
                                                    float *__restrict__ wgt) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return; /* uniform per wavefront */
  constexpr int MAXV = 16; /* E <= 1024 */
  float p[MAXV];
  const float *lg = logits + (size_t)t * E;
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int e = lane + 64 * i;
    p[i] = e < E ? lg[e] : -INFINITY;
    mx = fmaxf(mx, p[i]);
  }
  mx = hipq_group_max<64>(mx);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int e = lane + 64 * i;
    p[i] = e < E ? (float)exp((double)(p[i] - mx)) : 0.f;
    sum += p[i];
  }
  sum = hipq_group_sum<64>(sum);
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int e = lane + 64 * i;
    p[i] = e < E ? __fdiv_rn(p[i], sum) : -1.f; /* -1: never selected */
  }
  float ksum = 0.f;
  float myw = 0.f; /* lane kk keeps the kk-th weight */
  int myi = 0;
  for (int kk = 0; kk < topk; ++kk) {
    float bv = -2.f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int e = lane + 64 * i;
      if (p[i] > bv) { /* ascending e within the lane: first maximum wins */
        bv = p[i];
        bi = e;
      }
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
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
  if (lane < topk) {
    idx[(size_t)t * topk + lane] = myi;
    wgt[(size_t)t * topk + lane] = renorm ? __fdiv_rn(myw, ksum) : myw;
  }
}

/* Count, scan and scatter of the (token, k) pairs by expert in one workgroup:
 * the sort of a decode step or a short prefill chunk is a few thousand pairs, and
 * four tiny launches would cost more than the work. E <= 1024. */
__global__ __launch_bounds__(1024) void sort_pairs_kernel(const int32_t *__restrict__ idx, int P,
                                                          int E, int *__restrict__ offsets,
                                                          int *__restrict__ slot_pair,
                                                          int *__restrict__ pair_slot) {
  __shared__ int cnt[1024];
  __shared__ int off[1024];
  const int t = threadIdx.x;
  cnt[t] = 0;
  __syncthreads();
  for (int i = t; i < P; i += 1024) atomicAdd(&cnt[idx[i]], 1);
  __syncthreads();
  /* inclusive scan over the 1024 slots (Hillis-Steele), exclusive = inclusive - own */
  const int own = cnt[t];
  off[t] = own;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int v = t >= d ? off[t - d] : 0;
    __syncthreads();
    off[t] += v;
    __syncthreads();
  }
  const int excl = off[t] - own;
  if (t < E) offsets[t] = excl;
  if (t == E - 1) offsets[E] = off[t];
  __syncthreads();
  off[t] = excl;
  cnt[t] = 0;
  __syncthreads();
  for (int i = t; i < P; i += 1024) {
    const int e = idx[i];
    const int slot = off[e] + atomicAdd(&cnt[e], 1);
    slot_pair[slot] = i;
    pair_slot[i] = slot;
  }
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
                            int *__restrict__ cursor) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = acc;
      acc += counts[e];
      cursor[e] = 0;
    }
    offsets[E] = acc;
  }
}

__global__ void scatter_kernel(const int32_t *__restrict__ idx, int P,
                               const int *__restrict__ offsets, int *__restrict__ cursor,
                               int *__restrict__ slot_pair, int *__restrict__ pair_slot) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P) return;
  const int e = idx[i];
  const int slot = offsets[e] + atomicAdd(&cursor[e], 1);
  slot_pair[slot] = i;
  pair_slot[i] = slot;
}

__device__ __forceinline__ float silu_ref(float g) {
  /* sigmoid in double on the float-rounded exponential, as the reference */
  const float en = (float)exp((double)(-g));
  const float sig = (float)(1.0 / (1.0 + (double)en));
  return sig * g;
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
                                                      int I, float *__restrict__ h) {
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
        h[(size_t)(s0 + g.r) * I + col0 + g.g] = silu_ref(g.v) * u.v;
    }
  }
}

/* contrib[slot][col] = (h_slot . Wdown[e][col]) * weight(pair); same structure */
template <int DT, int T, int KC, int G, int CPW>
__global__ __launch_bounds__(256) void down_kernel(const WView *__restrict__ views, int E_, QView hq,
                                                   const int *__restrict__ offsets,
                                                   const int *__restrict__ slot_pair,
                                                   const float *__restrict__ wgt, int H,
                                                   float *__restrict__ contrib) {
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
        contrib[(size_t)(s0 + o.r) * H + col0 + o.g] = o.v * wgt[slot_pair[s0 + o.r]];
    }
  }
}

/* The same two products for rows longer than one chunk (K > 4096): one engine call
 * per column group, no cross-group prefetch. */
template <int DT>
__global__ __launch_bounds__(256) void gate_up_long_kernel(const WView *__restrict__ views, int E_,
                                                           QView xq, const int *__restrict__ offsets,
                                                           const int *__restrict__ slot_pair,
                                                           int topk, int I, float *__restrict__ h) {
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
      h[(size_t)(s0 + g.r) * I + col0 + g.g] = silu_ref(g.v) * u.v;
  }
}

template <int DT>
__global__ __launch_bounds__(256) void down_long_kernel(const WView *__restrict__ views, int E_,
                                                        QView hq, const int *__restrict__ offsets,
                                                        const int *__restrict__ slot_pair,
                                                        const float *__restrict__ wgt, int H,
                                                        float *__restrict__ contrib) {
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
      contrib[(size_t)(s0 + o.r) * H + col0 + o.g] = o.v * wgt[slot_pair[s0 + o.r]];
  }
}

/* y[t][c] = sum of the token's contributions, ascending expert id */
__global__ __launch_bounds__(256) void combine_kernel(const int32_t *__restrict__ idx,
                                                      const int *__restrict__ pair_slot, int topk,
                                                      int H, const float *__restrict__ contrib,
                                                      float *__restrict__ y) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= H) return;
  int ord[32];
  for (int k = 0; k < topk; ++k) ord[k] = k;
  for (int a = 1; a < topk; ++a) { /* insertion sort by expert id */
    const int v = ord[a];
    const int ev = idx[(size_t)t * topk + v];
    int b = a - 1;
    while (b >= 0 && idx[(size_t)t * topk + ord[b]] > ev) {
      ord[b + 1] = ord[b];
      --b;
    }
    ord[b + 1] = v;
  }
  float acc = 0.f;
  for (int k = 0; k < topk; ++k) {
    const int slot = pair_slot[t * topk + ord[k]];
    acc = acc + contrib[(size_t)slot * H + c];
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
void launch_gate_up(const hipq_moe_desc &d, const WView *views, const QAct &xq, const MoeBufs &b,
                    hipStream_t s) {
  const size_t lds = 4 * GemvLds<DT, RTOK, G, false>::DWORDS * sizeof(uint32_t);
  if (d.hidden > KC) {
    const dim3 grid((d.intermediate + 7) / 8, d.experts);
    const size_t lds_long = 4 * GemvLds<DT, RTOK, 2, false>::DWORDS * sizeof(uint32_t);
    hipLaunchKernelGGL((gate_up_long_kernel<DT>), grid, dim3(256), lds_long, s, views, d.experts,
                       qview(xq), b.offsets, b.slot_pair, d.topk, d.intermediate, b.h);
    return;
  }
  const dim3 grid((d.intermediate + 4 * G * CPW - 1) / (4 * G * CPW), d.experts);
  hipLaunchKernelGGL((gate_up_kernel<DT, T, KC, G, CPW>), grid, dim3(256), lds, s, views, d.experts,
                     qview(xq), b.offsets, b.slot_pair, d.topk, d.intermediate, b.h);
}
template <int DT, int T, int KC, int G>
void launch_down(const hipq_moe_desc &d, const WView *views, const QAct &hq, const MoeBufs &b,
                 hipStream_t s) {
  const size_t lds = 4 * GemvLds<DT, RTOK, G, false>::DWORDS * sizeof(uint32_t);
  if (d.intermediate > KC) {
    const dim3 grid((d.hidden + 7) / 8, d.experts);
    const size_t lds_long = 4 * GemvLds<DT, RTOK, 2, false>::DWORDS * sizeof(uint32_t);
    hipLaunchKernelGGL((down_long_kernel<DT>), grid, dim3(256), lds_long, s, views, d.experts,
                       qview(hq), b.offsets, b.slot_pair, b.wgt, d.hidden, b.contrib);
    return;
  }
  const dim3 grid((d.hidden + 4 * G * CPW - 1) / (4 * G * CPW), d.experts);
  hipLaunchKernelGGL((down_kernel<DT, T, KC, G, CPW>), grid, dim3(256), lds, s, views, d.experts,
                     qview(hq), b.offsets, b.slot_pair, b.wgt, d.hidden, b.contrib);
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
  const WView *views;
  const QAct &xq;
  const MoeBufs &b;
  hipStream_t s;
  template <int T, int KC, int G> void operator()() const { launch_gate_up<DT, T, KC, G>(d, views, xq, b, s); }
};
template <int DT> struct DownLauncher {
  const hipq_moe_desc &d;
  const WView *views;
  const QAct &hq;
  const MoeBufs &b;
  hipStream_t s;
  template <int T, int KC, int G> void operator()() const { launch_down<DT, T, KC, G>(d, views, hq, b, s); }
};

template <int DT>
int launch_grouped(const hipq::MoeArgs *a, const MoeBufs &b, const WView *views, const QAct &xq,
                   const QAct &hq, hipStream_t s) {
  const hipq_moe_desc &d = a->desc;
  const int64_t P = (int64_t)d.tokens * d.topk;
  int rc;
  for_row_length<DT>(d.hidden, GateUpLauncher<DT>{d, views, xq, b, s});
  HIPQ_HIP(hipGetLastError());
  if (DT == HIPQ_Q4_0)
    rc = hipq::launch_quantize_q8_0(b.h, P, d.intermediate, d.intermediate, &hq, nullptr, s);
  else
    rc = hipq::launch_quantize_q8_K(b.h, P, d.intermediate, d.intermediate, 0, &hq, nullptr, s);
  if (rc) return rc;
  for_row_length<DT>(d.intermediate, DownLauncher<DT>{d, views, hq, b, s});
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace

namespace hipq {

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
    hipLaunchKernelGGL(router_logits_kernel, dim3(T), dim3(256), 0, s, a->x, a->router_weight,
                       d.hidden, E, b.logits);
    HIPQ_HIP(hipGetLastError());
    logits = b.logits;
  }
  int32_t *idx = a->topk_idx ? a->topk_idx : b.idx;
  float *wgt = a->topk_w ? a->topk_w : b.wgt;
  hipLaunchKernelGGL(route_kernel, dim3((T + 3) / 4), dim3(256), 0, s, logits, T, E, d.topk,
                     d.renormalize, idx, wgt);
  HIPQ_HIP(hipGetLastError());
  b.wgt = wgt;
  if (P <= 16384 && E <= 1024) {
    hipLaunchKernelGGL(sort_pairs_kernel, dim3(1), dim3(1024), 0, s, idx, P, E, b.offsets, b.slot_pair,
                       b.pair_slot);
  } else {
    hipLaunchKernelGGL(fill_int_kernel, dim3((E + 255) / 256), dim3(256), 0, s, b.counts, E, 0);
    hipLaunchKernelGGL(count_kernel, dim3((P + 255) / 256), dim3(256), 0, s, idx, P, b.counts);
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(64), 0, s, b.counts, E, b.offsets, b.cursor);
    hipLaunchKernelGGL(scatter_kernel, dim3((P + 255) / 256), dim3(256), 0, s, idx, P, b.offsets,
                       b.cursor, b.slot_pair, b.pair_slot);
  }
  HIPQ_HIP(hipGetLastError());

  QAct xq = qact_carve(is_k, b.xq_mem, T, d.hidden);
  QAct hq = qact_carve(is_k, b.hq_mem, P, d.intermediate);
  int rc = is_k ? launch_quantize_q8_K(a->x, T, d.hidden, d.hidden, 0, &xq, nullptr, s)
                : launch_quantize_q8_0(a->x, T, d.hidden, d.hidden, &xq, nullptr, s);
  if (rc) return rc;
  if (dt == HIPQ_Q4_0)
    rc = launch_grouped<HIPQ_Q4_0>(a, b, views, xq, hq, s);
  else if (dt == HIPQ_Q4_K)
    rc = launch_grouped<HIPQ_Q4_K>(a, b, views, xq, hq, s);
  else
    rc = launch_grouped<HIPQ_Q6_K>(a, b, views, xq, hq, s);
  if (rc) return rc;
  hipLaunchKernelGGL(combine_kernel, dim3((d.hidden + 255) / 256, T), dim3(256), 0, s, idx,
                     b.pair_slot, d.topk, d.hidden, b.contrib, a->y);
  HIPQ_HIP(hipGetLastError());
  return HIPQ_OK;
}

} // namespace hipq
