/* SPDX-License-Identifier: Apache-2.0 */
/**
 * @file   hipq.h
 * @brief  C ABI of the MI355X (gfx950) quantized-weight matmul back-end.
 *
 * One shared library (libhipq.so) exports exactly these symbols. Signatures use
 * plain pointers and sizes only. Every function returns 0 on success or a
 * negative hipq_status and never throws; hipq_last_error() gives the message
 * of the calling thread's last failure. All entry points may be called from
 * several host threads at once (the reference's MoE layer calls its matmul
 * from inside an OpenMP loop).
 *
 * Reference interfaces replaced (paths relative to the reference checkout):
 *   nntrainer/tensor/cpu_backend/cpu_backend.h:937-1165  (gemm_q4_0, gemm_q4_K,
 *       gemm_q6_K, quantize_q4_0/q4_K/q6_K, repack_q4_0/q4_K, init_backend)
 *   nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface.h:28-342
 *   nntrainer/tensor/float_tensor.cpp:923-969            (dotQnK dispatch)
 *   Applications/CausalLM/layers/qwen_moe_layer.cpp:394-503 (MoE block)
 *
 * Memory: `mem` says where the caller's buffers live. HIPQ_MEM_DEVICE buffers are
 * device pointers; the call only enqueues work on `stream` and returns.
 * HIPQ_MEM_HOST buffers are ordinary host memory; the call copies in, runs,
 * copies out and returns when the result is in the host buffer. A call of a
 * few rows (a decode step or a short chunk: up to 128 rows, at most 2 MiB a side) uses no
 * copy engine: a kernel reads the rows from page-locked memory (memory of
 * hipq_host_alloc as it is, other memory through a page-locked staging buffer),
 * the product kernels write the outputs there, and the call returns when the
 * last kernel has set a flag in page-locked memory.
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 */
#ifndef HIPQ_H
#define HIPQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define HIPQ_API __attribute__((visibility("default")))
#else
#define HIPQ_API
#endif

typedef enum hipq_status {
  HIPQ_OK = 0,
  HIPQ_ERR_INVALID_ARGUMENT = -1, /* bad dims / null pointer / unknown enum  */
  HIPQ_ERR_NOT_INITIALIZED = -2,  /* hipq_init has not succeeded             */
  HIPQ_ERR_RUNTIME = -3,          /* a HIP call failed (message has details) */
  HIPQ_ERR_NOT_SUPPORTED = -4,    /* valid request this build cannot serve   */
  HIPQ_ERR_OUT_OF_MEMORY = -5
} hipq_status;

/** Weight formats; values are the ggml type ids the reference uses
 *  (nntr_ggml_impl_common.h:166-176). */
typedef enum hipq_dtype { HIPQ_Q4_0 = 2, HIPQ_Q4_K = 12, HIPQ_Q6_K = 14 } hipq_dtype;

/** Byte layout of weights handed to hipq_weight_create.
 *  CANONICAL: rows of plain ggml blocks (block_q4_0 18 B / block_q4_K 144 B /
 *             block_q6_K 210 B), row n = output column n (W^T, N x K).
 *  X8:        the 8-row interleave NNTrainer stores in its tensors and model
 *             files for Q4_0 and Q4_K (repack_q4_0 / repack_q4_K,
 *             nntr_ggml_impl.cpp:8189-8245). Not defined for Q6_K. */
typedef enum hipq_layout { HIPQ_LAYOUT_CANONICAL = 0, HIPQ_LAYOUT_X8 = 1 } hipq_layout;

typedef enum hipq_mem { HIPQ_MEM_HOST = 0, HIPQ_MEM_DEVICE = 1 } hipq_mem;

/** Which of the reference's two Q8_K activation quantizers to reproduce.
 *  ROW: quantize_row_q8_K (nntr_ggml_impl_quant.cpp:1334-1374) -- used for
 *       M == 1, for leftover rows M % 4 and for every Q6_K row.
 *  MAT: per-row content of quantize_mat_q8_K_4x8 (nntr_ggml_impl.cpp:7504-7737)
 *       -- used for rows [0, 4*(M/4)) of a Q4_K matmul with M > 1.
 *  They differ only in rare roundings and in the sign convention when +amax and
 *  -amax both occur. */
typedef enum hipq_q8k_variant { HIPQ_Q8K_ROW = 0, HIPQ_Q8K_MAT = 1 } hipq_q8k_variant;

/** Opaque device-resident weight matrix. */
typedef struct hipq_weight *hipq_weight_t;

/** Replaces init_backend() (x86_compute_backend.cpp:31): selects the GPU and
 *  creates the library state. Idempotent for the same device. */
HIPQ_API int hipq_init(int device);
/** Frees every cached buffer. Weights must be destroyed first. */
HIPQ_API int hipq_shutdown(void);
HIPQ_API const char *hipq_last_error(void);
/** Library version, "major.minor". */
HIPQ_API const char *hipq_version(void);

/** Bytes of an N x K weight matrix in canonical or x8 form (same size), or a
 *  negative status when K is not a multiple of the block size (32 for Q4_0,
 *  256 for Q4_K / Q6_K; q4_0_tensor.cpp:25-28, q4_k_tensor.cpp:23-27). */
HIPQ_API int64_t hipq_weight_nbytes(int dtype, int64_t N, int64_t K);

/** Uploads a weight matrix and re-lays it out once for the GPU kernels
 *  (structure-of-arrays: quants, scales and headers in separate 16-byte-aligned
 *  planes). `bytes` may be host or device memory (`mem`). The handle is what
 *  FullyConnectedLayer's weight tensor becomes on this back-end. */
HIPQ_API int hipq_weight_create(int dtype, int layout, int64_t N, int64_t K,
                                const void *bytes, int mem, hipq_weight_t *out);
/** Waits for the device, then frees the weight. A HIP graph captured from a call that named
 *  the weight (a matmul on it, an MoE block it is an expert of) must not be replayed
 *  afterwards. */
HIPQ_API int hipq_weight_destroy(hipq_weight_t w);
HIPQ_API int hipq_weight_dims(hipq_weight_t w, int *dtype, int64_t *N, int64_t *K);

/** One tensor of a weight file in NNTrainer's MODEL_FORMAT_BIN: the file is the
 *  tensors of the model's graph one after the other with no directory, so the
 *  caller lists them in graph order (NeuralNetwork::load,
 *  models/neuralnet.cpp:679-712). dtype HIPQ_Q4_0 / HIPQ_Q4_K / HIPQ_Q6_K: an
 *  N x K weight this library takes (its size follows from the dims; a Q4_K
 *  tensor is preceded by its 16-bit quantization scheme, Q4_0 and Q6_K tensors
 *  are not, neuralnet.cpp:696-703). dtype HIPQ_FILE_SKIP: `bytes` bytes of
 *  something else (fp32 norms, embeddings, biases). */
#define HIPQ_FILE_SKIP (-1)
typedef struct hipq_file_tensor {
  int dtype;
  int layout; /* hipq_layout of a weight; NNTrainer writes Q4_0 and Q4_K as X8 */
  int64_t N, K;
  int64_t bytes; /* HIPQ_FILE_SKIP only */
} hipq_file_tensor;
/** Where each listed tensor's data starts (after a Q4_K tensor's scheme word)
 *  when the first one starts at `offset`, and where the list ends. Host
 *  arithmetic only: usable without a device. data_offsets may be NULL. */
HIPQ_API int hipq_file_layout(int count, const hipq_file_tensor *tensors, int64_t offset,
                              int64_t *data_offsets, int64_t *end_offset);
/** Reads the listed tensors from `path` starting at `offset` and creates a
 *  weight handle for each quantized one (out[i] = NULL for skipped tensors).
 *  On an error no handle is left behind. A Q4_K tensor whose scheme word says
 *  Q4_Kx8 (quantizer.h:37) must be listed with HIPQ_LAYOUT_X8. */
HIPQ_API int hipq_weights_from_file(const char *path, int64_t offset, int count,
                                    const hipq_file_tensor *tensors, hipq_weight_t *out,
                                    int64_t *end_offset);

/** Activation quantizer fp32 -> Q8_0, canonical block_q8_0 output (34 B per 32
 *  values), M rows of K values (K % 32 == 0). Replaces nntr_quantize_row_q8_0 /
 *  nntr_quantize_mat_q8_0_4x8 (nntr_ggml_impl_quant.cpp:532-875,
 *  nntr_ggml_impl.cpp:7788-8012), whose per-row content is identical. */
HIPQ_API int hipq_quantize_q8_0(const float *A, int64_t M, int64_t K, int64_t lda,
                                void *out_blocks, int mem, void *stream);
/** Activation quantizer fp32 -> Q8_K, canonical block_q8_K output (292 B per
 *  256 values: fp32 d, 256 int8, 16 int16 group sums), K % 256 == 0. */
HIPQ_API int hipq_quantize_q8_K(const float *A, int64_t M, int64_t K, int64_t lda,
                                int variant, void *out_blocks, int mem, void *stream);

/** C[M x N] = A[M x K] . W^T with on-the-fly activation quantization; the GPU
 *  form of gemm_q4_0 / gemm_q4_K / gemm_q6_K (x86_compute_backend.cpp:301-341)
 *  as reached from FloatTensor::dotQnK (float_tensor.cpp:923-969). M == 1 runs
 *  the decode GEMV kernels, M > 1 the prefill GEMM kernels. lda >= K and
 *  ldc >= N are row strides in elements. With M == 1, K <= 4096, N < 32768 and
 *  device memory the call is a single kernel launch (the GEMV quantizes the row
 *  itself) and uses no workspace.
 *  Outputs carry the bits of the reference's AVX2 kernels for every Q4_0 product and for
 *  Q4_K with up to 8 rows (up to 16 against 1024 columns or more, up to 64 where
 *  columns / 32 x rows / 8 x K / 256 <= 8192, once the weight's copy described below exists
 *  or may be made) and Q6_K with up to 16 rows (up to 8 for matrices
 *  of 2^24 weights or more, up to 4 from 2^25, up to 2 from 2^28: there the matrix cores are
 *  faster, up to several times); with more rows the K-formats run on the
 *  int8 matrix cores and agree with the reference to 1e-4 of the output's maximum (same
 *  quantized activations, another order of the fp32 sums). The first such product of a
 *  weight adds a copy of it in the kernels' load order (allocates; 0.56 bytes per weight
 *  for Q4_K, 0.875 for Q6_K), kept until hipq_weight_destroy. Q4_K with 5..16 rows and 1024
 *  columns or more (4 rows from 4096, 3 from 8192 columns) reads the same copy: those row
 *  counts run on the matrix cores as well, with the reference's bits (a batch of decode
 *  rows against a 12288 x 4096 matrix: 11 us for eight, 14 us for sixteen, 8 us for one).
 *  Q4_0 has the same kind of kernel for a few rows (gemm_rows_q40.hip, off the weight as it is
 *  stored: eight rows against 12288 x 4096 in 11 us, against 151936 x 1024 in 26 us); every Q4_0
 *  kernel carries the reference's bits, so there the row count only selects the fastest. */
HIPQ_API int hipq_matmul(hipq_weight_t w, const float *A, int64_t M, int64_t lda,
                         float *C, int64_t ldc, int mem, void *stream);

/** `rows` independent one-row products in one call: row r of C = row r of A . W^T with the bits
 *  of hipq_matmul(w, A + r * lda, 1, ...). Replaces the loop over batch entries of a decode step,
 *  FullyConnectedLayer::incremental_forwarding with to - from == 1 (fc_layer.cpp:266-296: one
 *  input_step.dot(weight, hidden_step) per entry, each an M = 1 product). It differs from
 *  hipq_matmul with M = rows for Q4_K only, where the reference quantizes rows it multiplies
 *  together four at a time and sums their sub-block pairs separately; rows of different batch
 *  entries are never multiplied together there. The rows share one pass over the weights (Q4_K
 *  against 1024 columns or more: on the matrix cores, gemm_rows_q4k.hip; Q4_0: whatever
 *  hipq_matmul picks for that many rows) and, with host memory, one transfer each way. */
HIPQ_API int hipq_matmul_each_row(hipq_weight_t w, const float *A, int64_t rows, int64_t lda,
                                  float *C, int64_t ldc, int mem, void *stream);

/** hipq_matmul on device buffers for callers that cannot allocate device memory:
 *  code under HIP graph capture, tight serving loops, harnesses that forbid it.
 *  It has no counterpart in the reference. The quantized activations of the call
 *  live in a fixed array inside the library's device code (32 MiB; each GPU the
 *  library runs on holds one until the process ends) instead of the per-stream
 *  workspace that hipq_matmul grows on demand. The array has four slots of 8 MiB,
 *  one for each of the first four streams that use this entry point (a fifth stream
 *  gets HIPQ_ERR_NOT_SUPPORTED until hipq_stream_release has given a slot back), so calls
 *  on different streams do not share memory; calls on ONE stream run in order and share
 *  its slot, which keeps the last call's contents. A call that needs more than a slot
 *  (M * K beyond about 3.9 million values for Q6_K weights, 7 million for Q4_0
 *  and Q4_K) returns HIPQ_ERR_NOT_SUPPORTED. The call performs no device
 *  allocation and no free and enqueues the same kernels as hipq_matmul, so
 *  results are the same bits wherever the same kernel runs. Where the two may take
 *  different kernels: a weight that has no tile copy yet (only an allocating call builds
 *  one) goes through the GEMV engine here, which carries the reference's bits where
 *  hipq_matmul's matrix-core product agrees to 1e-4; and a Q4_K or Q6_K product of up to
 *  128 rows that hipq_matmul forms in parts of K takes whole rows here when the parts'
 *  partial sums do not fit the slot beside the activations, or when C is not 16-byte
 *  aligned with ldc a multiple of four (both entry points then): the fp32 sums then have
 *  another order, within the 1e-4 of every matrix-core product. Results of the K-formats'
 *  matrix-core products are therefore stable to the tolerance, not to the bit, across ldc,
 *  alignment and entry point. */
HIPQ_API int hipq_matmul_noalloc(hipq_weight_t w, const float *A, int64_t M, int64_t lda,
                                 float *C, int64_t ldc, void *stream);

/** One fp32 activation against several weights sharing K (the QKV layer's
 *  vector dot, float_tensor.cpp:724-798): quantizes A once. One row against up to
 *  four weights of one format (K <= 4096, fewer than 32768 rows together, device
 *  memory) is a single kernel launch for all of them. With more than 8 rows the Q4_0
 *  and the Q4_K products go out four weights a launch as well (the column tiles of the
 *  weights side by side in one grid), after the one quantization; so do two or more Q4_0 or
 *  Q4_K weights with 2 to 16 rows (a decode step of a batch; to 64 rows on narrow weights),
 *  through the few-rows kernels, with the reference's bits. Every output equals what
 *  hipq_matmul gives for that weight alone bit for bit, except where the single call of a
 *  Q4_K weight takes the prefill GEMM for those rows (then to 1e-4, as every product of that
 *  kernel). */
HIPQ_API int hipq_matmul_multi(int count, const hipq_weight_t *w, const float *A,
                               int64_t M, int64_t lda, float *const *C,
                               const int64_t *ldc, int mem, void *stream);

/** The first half of a gated MLP: out[M x N] = swiglu(A . W_act^T, A . W_mul^T) with the
 *  framework's swiglu, X = (Y / (1 + exp(-Y))) * Z in fp32 (nntrainer::swiglu,
 *  fallback_internal.cpp:417-423). In the LLM application these are three layers, the FCs
 *  "ffn_up" (Y) and "ffn_gate" (Z) and the SwiGLULayer on their outputs
 *  (Applications/CausalLM/layers/swiglu.cpp:40-62, causal_lm.cpp:672-695); here one call that
 *  quantizes A once, and for one row (K <= 4096, 2 N < 32768, device memory) one kernel launch
 *  in which the two products never leave the registers. The products are those of hipq_matmul
 *  bit for bit; the exponential is the device's expf. */
HIPQ_API int hipq_mlp_swiglu(hipq_weight_t w_act, hipq_weight_t w_mul, const float *A, int64_t M,
                             int64_t lda, float *out, int64_t ldo, int mem, void *stream);

/** The whole gated MLP of a decoder layer: out[M x Nd] = swiglu(A . W_act^T, A . W_mul^T) . W_down^T,
 *  the four layers "ffn_up", "ffn_gate", "swiglu" and "ffn_down" of CausalLM::createMlp
 *  (Applications/CausalLM/causal_lm.cpp:671-705) as one call. The hidden activation [M x N] stays in
 *  device memory between the gated half and the down projection: with host operands only A goes in
 *  and only out comes back, where the two calls (hipq_mlp_swiglu, hipq_matmul) move the hidden rows
 *  out and in again and wait once more. W_down has K = N of the other two. Every value equals what
 *  those two calls give bit for bit (the same kernels on the same operands). */
HIPQ_API int hipq_mlp_swiglu_down(hipq_weight_t w_act, hipq_weight_t w_mul, hipq_weight_t w_down,
                                  const float *A, int64_t M, int64_t lda, float *out, int64_t ldo,
                                  int mem, void *stream);

/** Mixture-of-experts feed-forward block (MoELayer::incremental_forwarding,
 *  qwen_moe_layer.cpp:394-503): softmax over E router logits, top-k, weights
 *  renormalised to sum 1, per (token, expert) SwiGLU MLP
 *  down(silu(gate(x)) * up(x)), outputs combined in ascending expert order.
 *  Tokens are sorted by expert on the device and each projection is one grouped
 *  launch over the active experts. */
typedef struct hipq_moe_desc {
  int32_t tokens;       /* T                                   */
  int32_t hidden;       /* H, K of gate/up, N of down          */
  int32_t intermediate; /* I, N of gate/up, K of down          */
  int32_t experts;      /* E                                   */
  int32_t topk;         /* experts per token                   */
  int32_t renormalize;  /* 1: divide top-k weights by their sum (incremental
                           path); 0: use softmax values as is (forwarding path,
                           qwen_moe_layer.cpp:161-259)           */
} hipq_moe_desc;

/** gate/up/down: E handles each. x [T x H]. Exactly one of `router_logits`
 *  [T x E] (logits already computed) and `router_weight` [H x E] fp32 (the
 *  layer's "gate" weight; logits = x . router_weight) must be non-NULL.
 *  y [T x H]. topk_idx [T x topk] int32 and topk_w [T x topk] fp32 are optional
 *  outputs of the routing.
 *  The first call with a set of Q4_K experts re-stores them on the device in the
 *  order the expert kernels read (a one-time pass, synchronous); from then on
 *  these handles serve hipq_moe_forward only and hipq_matmul refuses them. In
 *  the reference an expert's weight tensors belong to its MoE layer alone
 *  (qwen_moe_layer.cpp:50-159). */
HIPQ_API int hipq_moe_forward(const hipq_moe_desc *desc, const hipq_weight_t *gate,
                              const hipq_weight_t *up, const hipq_weight_t *down,
                              const float *x, const float *router_logits,
                              const float *router_weight, float *y,
                              int32_t *topk_idx, float *topk_w, int mem,
                              void *stream);

/** Variants of the block for the other MoE layers of the LLM application. All pointers
 *  live where `mem` says, like x.
 *  - HIPQ_MOE_QWEN (or ext == NULL): hipq_moe_forward as above. It also serves the cached
 *    layer (CachedSlimMoELayer::incremental_forwarding, qwen_moe_layer_cached.cpp:266-470):
 *    that layer differs in where expert weights live between calls (paged in on demand, 32 kept;
 *    here all experts stay in HBM) and in running one batched product per expert, which is how
 *    this library runs every MoE; routing, expert arithmetic and the ascending-expert sum are
 *    the same.
 *    Against the cached layer's own arithmetic (rows [0, 4*(n/4)) of an expert's n tokens through
 *    the 4-row quantizer and GEMM order, nntrainer::swiglu with the x86 back-end's approximate
 *    exponential for n > 1) the outputs agree to 1e-4 of the largest, not to the bit: every
 *    (token, expert) pair here has the bits of its own M = 1 products.
 *  - HIPQ_MOE_GPT_OSS: GptOssMoELayer (gpt_oss_moe_layer.cpp:372-449, 452-568): the router
 *    logits take router_bias [E]; per expert g = gate(x) + gate_bias[e], u = up(x) + up_bias[e],
 *    h = (g / (1 + exp(-alpha g))) * (u + 1), y_e = down(h) + down_bias[e]; top-k weights
 *    renormalised per desc->renormalize. `limit` > 0 clamps the biased pre-activations first,
 *    g = min(g, limit), u = min(max(u, -limit), limit): the cached layer does so with limit 7
 *    (gpt_oss_moe_layer_cached.cpp:497-507, gpt_oss_moe_layer_cached.h:137), the uncached
 *    one has the same two lines commented out (gpt_oss_moe_layer.cpp:414, 419) and passes 0. */
enum { HIPQ_MOE_QWEN = 0, HIPQ_MOE_GPT_OSS = 1 };
typedef struct hipq_moe_ext {
  int32_t variant;          /* HIPQ_MOE_*                                    */
  float alpha;              /* gpt_oss: 1.702 (gpt_oss_moe_layer.h:126)      */
  const float *router_bias; /* [E] or NULL; needs router_weight              */
  const float *gate_bias;   /* [E x I], gpt_oss                              */
  const float *up_bias;     /* [E x I], gpt_oss                              */
  const float *down_bias;   /* [E x H], gpt_oss                              */
  float limit;              /* gpt_oss: 0 = no clamp, > 0 as above           */
  int32_t biases_on_device; /* non-zero: the four bias pointers are device memory
                               whatever `mem` says (a layer uploads them once,
                               hipq_device_alloc / hipq_device_upload)         */
  int32_t router_on_device; /* non-zero: router_weight is device memory whatever
                               `mem` says (1 MB at 2048 x 128: not worth a copy
                               per call)                                       */
} hipq_moe_ext;
HIPQ_API int hipq_moe_forward_ext(const hipq_moe_desc *desc, const hipq_moe_ext *ext,
                                  const hipq_weight_t *gate, const hipq_weight_t *up,
                                  const hipq_weight_t *down, const float *x,
                                  const float *router_logits, const float *router_weight,
                                  float *y, int32_t *topk_idx, float *topk_w, int mem,
                                  void *stream);

/** Device memory for a caller that has no HIP runtime of its own (the framework plug-in keeps
 *  the biases of a GPT-OSS block and activations that stay on the GPU between two of its layers
 *  in it). No counterpart in the reference: its tensors are host memory only. upload / download
 *  are ordered on `stream` and return when the host bytes have been read / written. */
HIPQ_API int hipq_device_alloc(void **ptr, size_t bytes);
HIPQ_API int hipq_device_free(void *ptr);
HIPQ_API int hipq_device_upload(void *dst_device, const void *src_host, size_t bytes, void *stream);
HIPQ_API int hipq_device_download(void *dst_host, const void *src_device, size_t bytes, void *stream);

/** Page-locked host memory, zero-filled: what a context's MemAllocator hands the framework's
 *  memory pool (MemAllocator::alloc / free, nntrainer/mem_allocator.cpp:22-30; set by the
 *  context, cl_context.cpp:83). Tensors that live in it cross to the GPU by DMA as they are
 *  (a prefill of 512 rows and more with 16 MiB of outputs in steps of 256 rows, a step's output
 *  leaving on a second stream of the library's while the next step's rows arrive and are
 *  multiplied; up to 128 rows of at most 2 MiB a side without a copy engine at all);
 *  any other host memory passed with HIPQ_MEM_HOST goes through a pinned staging ring inside
 *  the library (8 MiB), at the speed of a host memcpy. */
HIPQ_API int hipq_host_alloc(void **ptr, size_t bytes);
HIPQ_API int hipq_host_free(void *ptr);

/** Kernel timing without an external tracer. Between _begin and _end every kernel that calls of
 *  the SAME THREAD launch carries a start and a stop event of its own (attached to the dispatch:
 *  no marker packets between the kernels), up to max_launches of them. _end waits for the timed
 *  launches and returns how many there were (*count), and for the first `capacity` of them, in
 *  launch order, the kernel's own duration in milliseconds and the kernel as its launch site in
 *  this library's source names it (names may be NULL; the strings are literals of the library). What a kernel trace reports for the same launches. A launch
 *  that carries events delays the one behind it by a few microseconds, so the time of a whole call
 *  is taken without this switched on. No counterpart in the reference, whose profiler brackets
 *  host calls (nntrainer/utils/profiler.h). */
HIPQ_API int hipq_launch_timing_begin(int max_launches);
HIPQ_API int hipq_launch_timing_end(int capacity, int *count, float *ms, const char **names);

/** Frees the scratch the library keeps for a stream (it grows on demand with the calls made on
 *  the stream and is otherwise kept until hipq_shutdown) and gives back the stream's slot of the
 *  allocation-free entry point's array. Call it before destroying a stream
 *  that calls were made on; waits for the stream. When a call needs more scratch than the stream
 *  has, the library allocates a larger block (hipMalloc: not possible while the stream is being
 *  captured into a graph, so run a call of the largest shape once before capturing) and keeps the
 *  smaller one until a later call on the stream finds the stream drained. No counterpart in the reference, whose OpenCL
 *  back-end has one queue (opencl_command_queue_manager.cpp). */
HIPQ_API int hipq_stream_release(void *stream);

/** Offline weight quantizers fp32 [N x K] -> canonical blocks, on the GPU.
 *  Replace quantize_q4_0 / quantize_q4_K / quantize_q6_K
 *  (x86_compute_backend.cpp:343-370 -> nntr_ggml_impl_quant.cpp:452-467,
 *  1062-1077, 1274-1289). */
HIPQ_API int hipq_quantize_weights(int dtype, const float *W, int64_t N, int64_t K,
                                   void *out_blocks, int mem, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPQ_H */
