/* SPDX-License-Identifier: Apache-2.0 */
/*
 * nntr_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement, in plain C, of the arithmetic of NNTrainer's quantized-weight
 * matmul path (the "ggml interface" CPU back-end) as it behaves in an x86 AVX2
 * build made with GCC (the reference's own flags: -mavx2 -mfma, default
 * floating-point contraction). It exists so that the HIP kernels can be checked
 * against something that runs anywhere; it is never linked into, imported by or
 * used as a fallback for the product library. Only tests, the smoke check and
 * the CPU-baseline leg of the benchmark may load it.
 *
 * Every function names the reference file:line it follows. All paths are
 * relative to the reference checkout; GI = nntrainer/tensor/cpu_backend/
 * ggml_interface, IMPL = GI/nntr_ggml_impl.
 *
 * Pinning status (what each function has been checked against, see
 * tests/test_oracle_*.py): every function below is compared bit-for-bit
 * (bytes, or fp32 bit patterns) with the reference library built from the
 * reference sources (oracle/_ref) on seeded random and adversarial inputs, and
 * against closed forms (dequantize-and-dot in double, round trips, invariants).
 * The MoE block has no directly callable counterpart in the reference library
 * (the layer needs the whole framework); it is pinned by composing it from the
 * reference's own GEMV entry points and against a dense per-token evaluation.
 */
#ifndef NNTR_ORACLE_H
#define NNTR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Block sizes in bytes (IMPL/nntr_ggml_impl_common.h:72-150). */
#define ORC_QK_K 256
#define ORC_Q4_0_BYTES 18
#define ORC_Q8_0_BYTES 34
#define ORC_Q4_K_BYTES 144
#define ORC_Q6_K_BYTES 210
#define ORC_Q8_K_BYTES 292

/* IEEE binary16 <-> binary32 (IMPL/nntr_ggml_impl_fp16_fp32.cpp:69-79,165-220). */
float orc_fp16_to_fp32(uint16_t h);
uint16_t orc_fp32_to_fp16(float f);

/* Offline weight quantizers: src fp32 [nrow x k] row-major -> blocks row-major.
 * IMPL/nntr_ggml_impl_quant.cpp:382-418 (Q4_0), :901-979 (Q4_K), :1116-1186 (Q6_K). */
void orc_quantize_q4_0(const float *src, void *dst, int64_t nrow, int64_t k);
void orc_quantize_q4_K(const float *src, void *dst, int64_t nrow, int64_t k);
void orc_quantize_q6_K(const float *src, void *dst, int64_t nrow, int64_t k);

/* Dequantizers (closed forms of the block formats).
 * IMPL/nntr_ggml_impl_quant.cpp:469-494, 1079-1114, 1291-1325, 876-897, 1461-1471. */
void orc_dequantize_q4_0(const void *blocks, float *y, int64_t n);
void orc_dequantize_q4_K(const void *blocks, float *y, int64_t n);
void orc_dequantize_q6_K(const void *blocks, float *y, int64_t n);
void orc_dequantize_q8_0(const void *blocks, float *y, int64_t n);
void orc_dequantize_q8_K(const void *blocks, float *y, int64_t n);

/* x8 row interleave used for on-disk / in-tensor Q4_0 and Q4_K weights and its
 * inverse. IMPL/nntr_ggml_impl.cpp:8056-8158, 8189-8245. Return 0, or -1 when
 * nrow % 8 != 0 or k % 8 != 0 (same rule as the reference). */
int orc_repack_q4_0_x8(void *dst, const void *src, int64_t nrow, int64_t k);
int orc_unpack_q4_0_x8(void *dst, const void *src, int64_t nrow, int64_t k);
int orc_repack_q4_K_x8(void *dst, const void *src, int64_t nrow, int64_t k);
int orc_unpack_q4_K_x8(void *dst, const void *src, int64_t nrow, int64_t k);

/* Activation quantizers, output in canonical (de-interleaved) blocks.
 *  q8_0: IMPL/nntr_ggml_impl_quant.cpp:613-701 (AVX2 branch); the 4-row variant
 *        IMPL/nntr_ggml_impl.cpp:7879-7980 has identical per-row content.
 *  q8_K "row": IMPL/nntr_ggml_impl_quant.cpp:1334-1374 as GCC compiles it
 *        (iscale*x + magic contracted into one fused multiply-add).
 *  q8_K "mat": the 4-row AVX2 variant IMPL/nntr_ggml_impl.cpp:7504-7737
 *        (separately rounded product, positive-maximum sign rule). */
void orc_quantize_row_q8_0(const float *x, void *y, int64_t k);
void orc_quantize_row_q8_K(const float *x, void *y, int64_t k);
void orc_quantize_row_q8_K_mat(const float *x, void *y, int64_t k);
/* Canonical rows -> the reference's 4-row interleaved structures
 * (block_q8_0x4 / block_q8_Kx4), to compare bytes with the reference. */
void orc_interleave_q8_0x4(const void *rows4, void *dst, int64_t k);
void orc_interleave_q8_Kx4(const void *rows4, void *dst, int64_t k);

/* Matmuls C[M x N] = A[M x K] . W^T, W given as canonical blocks of N rows.
 * Control flow of GI/ggml_interface_omp.cpp:303-390 (Q4_0), :404-487 (Q4_K),
 * :500-566 (Q6_K); per-element fp32 evaluation order of the AVX2 kernels
 * IMPL/nntr_ggml_impl.cpp:9596-9761, 1080-3215 (Q4_0), :7094-7422, 5485-6992
 * (Q4_K), :8600-8695 (Q6_K). */
void orc_gemm_q4_0(int M, int N, int K, const float *A, const void *W, float *C);
void orc_gemm_q4_K(int M, int N, int K, const float *A, const void *W, float *C);
void orc_gemm_q6_K(int M, int N, int K, const float *A, const void *W, float *C);

/* Mixture-of-experts block, inference path with renormalised top-k weights.
 * Applications/CausalLM/layers/qwen_moe_layer.cpp:332-392, 394-503;
 * nntrainer/layers/acti_func.h:166-213, 286-288, 400-405;
 * nntrainer/tensor/float_tensor.cpp:1108-1180.
 *   x [T x H] fp32; logits [T x E] fp32 router logits (already x . gate);
 *   gate/up: E arrays of Q4_K blocks of [I x H]; down: E arrays of [H x I];
 *   y [T x H] fp32. topk_idx/topk_w (may be NULL) receive the routing. */
void orc_moe_forward(int kind /* 2 Q4_0, 12 Q4_K, 14 Q6_K */, int renormalize /* 0: the forwarding
                     path, qwen_moe_layer.cpp:161-259 */, int T, int H, int I, int E, int topk,
                     const float *x, const float *logits, const void *const *gate,
                     const void *const *up, const void *const *down, float *y, int32_t *topk_idx,
                     float *topk_w);
void orc_moe_forward_gpt_oss(int kind, int renormalize, int T, int H, int I, int E, int topk, const float *x,
                             const float *logits, const void *const *gate, const void *const *up,
                             const void *const *down, const float *gate_bias, const float *up_bias,
                             const float *down_bias, float alpha, float *y, int32_t *topk_idx,
                             float *topk_w);
void orc_moe_forward_q4_K(int T, int H, int I, int E, int topk, const float *x,
                          const float *logits, const void *const *gate,
                          const void *const *up, const void *const *down,
                          float *y, int32_t *topk_idx, float *topk_w);

void orc_swiglu(int64_t n, float *x, const float *y, const float *z);
/* nntrainer::swiglu as the x86 back-end evaluates it (table-and-cubic exponential, denormals
 * as zero): nntrainer/tensor/cpu_backend/x86/avx2_impl.cpp:227-316, 906-993. */
void orc_swiglu_x86(int64_t n, float *x, const float *y, const float *z);
void orc_swiglu_alpha_x86(int64_t n, float *x, const float *y, const float *z, float alpha);
/* The cached layers: one product per expert with M = its token count, swiglu by token count,
 * GPT-OSS with its clamps. qwen_moe_layer_cached.cpp:176-470, gpt_oss_moe_layer_cached.cpp:193-530.
 * Biases [E x I], [E x I], [E x H] (gpt_oss = 1 only). */
void orc_moe_forward_cached(int kind, int gpt_oss, int T, int H, int I, int E, int topk, const float *x,
                            const float *logits, const void *const *gate, const void *const *up,
                            const void *const *down, const float *gate_bias, const float *up_bias,
                            const float *down_bias, float alpha, float limit, float *y, int32_t *topk_idx,
                            float *topk_w);
void orc_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
