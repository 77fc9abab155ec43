// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hipq_host.h
 * @brief  C++ host core between the framework adapters (HipContext, FC and MoE
 *         layers) and the C ABI of libhipq (include/hipq.h).
 *
 * Nothing in here knows the framework's types. It provides
 *  - the translation of C-ABI status codes into the exceptions the framework
 *    uses on this path (std::invalid_argument for bad properties and
 *    dimensions, std::runtime_error for a failed kernel or dispatch,
 *    cf. nntrainer/tensor/cl_operations/blas_kernels.cpp:246-319, and
 *    nntrainer::exception::not_supported = a std::invalid_argument,
 *    nntrainer/nntrainer_error.h:157-159);
 *  - the device-side cache of weights keyed by the host pointer of the tensor
 *    the framework owns: layers may not allocate in finalize()
 *    (nntrainer/layers/layer_devel.h:187-189), so a weight is uploaded and put
 *    into the device layout the first time a forward call sees it;
 *  - the quantized matmul and the MoE block on host pointers.
 */
#ifndef HIPQ_HOST_H
#define HIPQ_HOST_H

#include <cstdint>
#include <atomic>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include <hipq.h>

namespace hipq_host {

/** raised for HIPQ_ERR_NOT_SUPPORTED; an invalid_argument like the framework's own */
struct not_supported : public std::invalid_argument {
  using std::invalid_argument::invalid_argument;
};

/** throws the exception that corresponds to a non-zero status code */
void check(int status, const char *what);

/**
 * Brings the device up once per process. Never throws: a machine without a
 * usable GPU leaves the runtime marked unavailable, as ClContext::initialize
 * does for a missing OpenCL device (nntrainer/cl_context.cpp:70-90).
 * @return true if kernels can be launched
 */
bool runtime_available(int device = 0) noexcept;

/** Layout of weight bytes as the framework hands them over. */
struct WeightSpec {
  int dtype;  /**< HIPQ_Q4_0 | HIPQ_Q4_K | HIPQ_Q6_K */
  int layout; /**< HIPQ_LAYOUT_X8 for Q4_0/Q4_K tensors of a loaded model
                   (ggml_interface.cpp:109-122), canonical for Q6_K */
  int64_t N;  /**< output features */
  int64_t K;  /**< input features  */
};

/** layout a framework tensor of this dtype uses for its bytes */
inline int framework_layout(int dtype) {
  return dtype == HIPQ_Q6_K ? HIPQ_LAYOUT_CANONICAL : HIPQ_LAYOUT_X8;
}

/**
 * Device copies of the weights, keyed by the host address of the bytes.
 * Thread safe: MoE calls its experts from an OpenMP loop
 * (Applications/CausalLM/layers/qwen_moe_layer.cpp:478-490) and weights are
 * read by one thread per node at load time (nntrainer/models/neuralnet.cpp:742-751).
 */
class WeightCache {
public:
  WeightCache() = default;
  ~WeightCache();
  WeightCache(const WeightCache &) = delete;
  WeightCache &operator=(const WeightCache &) = delete;

  /** the device weight for these host bytes; uploads on first use, and again when a
   *  sample of the bytes (first, last and six words in between) no longer matches the
   *  one taken at the upload: a buffer rewritten in place behind the layers' backs */
  hipq_weight_t get(const void *host_bytes, const WeightSpec &spec);
  /** forget (and free) the device copy of a host buffer whose content changed; the layers
   *  call it for their weights after the framework has read them from a file */
  void invalidate(const void *host_bytes);
  void clear();
  size_t size() const;
  /** counts the device copies this cache has freed: a handle taken from get() while the count read
   *  n is still alive as long as it reads n */
  uint64_t epoch() const { return freed.load(std::memory_order_acquire); }
  /** the sample get() compares (eight words of the buffer) */
  static uint64_t sample(const void *host_bytes, int64_t nbytes);

private:
  struct Entry {
    hipq_weight_t w;
    WeightSpec spec;
    uint64_t tag; /* sample of the host bytes at upload time */
  };
  mutable std::mutex mtx;
  std::unordered_map<const void *, Entry> map;
  std::atomic<uint64_t> freed{0};
};

/** The handles of a layer's many weights from its last call (a MoE layer's 3 x experts): a call finds
 *  them again by comparing each tensor's address and sample, without the cache's lock and hash look-up
 *  per weight (128 experts: 384 of them a call, which cost more than the rest of a decode step's host
 *  work). Valid while the cache has freed nothing since. */
struct HandleMemo {
  std::vector<const void *> bytes;
  std::vector<uint64_t> tags;
  std::vector<hipq_weight_t> w;
  uint64_t epoch = ~(uint64_t)0;
};

/** process-wide cache used by the layers */
WeightCache &global_cache();

/**
 * C[M x N] = A[M x K] * W^T with W given as quantized bytes in host memory;
 * A and C are host fp32. M == 1 runs the decode GEMV, M > 1 the prefill GEMM,
 * exactly the dispatch of FloatTensor::dotQnK
 * (nntrainer/tensor/float_tensor.cpp:923-969).
 */
void matmul(WeightCache &cache, const void *weight_bytes, const WeightSpec &spec,
            const float *A, int64_t M, int64_t lda, float *C, int64_t ldc);

/** `rows` one-row products against one weight in one call, each with the bits of matmul with
 *  M = 1: the batch entries of a decode step (fc_layer.cpp:266-296 loops over them) */
void matmul_each_row(WeightCache &cache, const void *weight_bytes, const WeightSpec &spec,
                     const float *A, int64_t rows, int64_t lda, float *C, int64_t ldc);

/** one activation against several weights (shared activation quantization),
 *  the vector overload of dot (float_tensor.cpp:724-798) */
void matmul_multi(WeightCache &cache, const std::vector<const void *> &weight_bytes,
                  const std::vector<WeightSpec> &specs, const float *A, int64_t M,
                  int64_t lda, const std::vector<float *> &C);

/** out[M x N] = swiglu(A . Wact^T, A . Wmul^T), both weights of one spec (hipq_mlp_swiglu) */
void mlp_swiglu(WeightCache &cache, const void *act_bytes, const void *mul_bytes, const WeightSpec &spec,
                const float *A, int64_t M, int64_t lda, float *out, int64_t ldo);
/** out[M x Nd] = swiglu(A . Wact^T, A . Wmul^T) . Wdown^T (hipq_mlp_swiglu_down): the hidden rows stay on the device */
void mlp_swiglu_down(WeightCache &cache, const void *act_bytes, const void *mul_bytes, const WeightSpec &spec,
                     const void *down_bytes, const WeightSpec &down_spec, const float *A, int64_t M, int64_t lda,
                     float *out, int64_t ldo);

struct MoeShape {
  int tokens, hidden, intermediate, experts, topk;
  bool renormalize;
};

/** What the GPT-OSS block adds to the Qwen block (hipq_moe_ext of include/hipq.h): host pointers,
 *  biases as [experts x intermediate], [experts x intermediate], [experts x hidden]. */
struct MoeExtras {
  bool gpt_oss = false;
  float alpha = 1.702f;
  float limit = 0.f; /* > 0: the cached layer's clamps on the biased gate and up values */
  const float *router_bias = nullptr;
  const float *gate_bias = nullptr, *up_bias = nullptr, *down_bias = nullptr;
  bool biases_on_device = false; /* the four pointers above are device copies (device_floats) */
  bool router_on_device = false; /* router_weight of the call is a device copy */
};

/** A device copy of n floats the caller owns; freed with device_release. */
float *device_floats(const float *host, size_t n);
void device_release(void *p) noexcept;

/** A device copy of a host tensor of floats that follows its source: made at the first get(),
 *  made again when the source's address, size or sampled content has changed. */
class DeviceMirror {
public:
  DeviceMirror() = default;
  ~DeviceMirror() { drop(); }
  DeviceMirror(const DeviceMirror &) = delete;
  DeviceMirror &operator=(const DeviceMirror &) = delete;
  const float *get(const float *host, size_t n);
  void drop() noexcept;

private:
  float *dev = nullptr;
  const float *src = nullptr;
  size_t count = 0;
  uint64_t tag = 0;
};

/** A device copy that the caller owns (not entered into a cache): for weights whose host bytes
 *  come and go (virtual tensors), where an address is no identity. */
hipq_weight_t upload(const void *host_bytes, const WeightSpec &spec);
void release(hipq_weight_t w) noexcept;

/**
 * The MoE block of qwen_moe_layer.cpp:394-503 on host pointers: router matmul
 * with the fp32 gate weight [hidden x experts], softmax, top-k, renormalise,
 * per-expert SwiGLU MLP on quantized weights, combine in ascending expert order.
 */
void moe_forward(WeightCache &cache, const MoeShape &shape, int dtype,
                 const std::vector<const void *> &gate_bytes,
                 const std::vector<const void *> &up_bytes,
                 const std::vector<const void *> &down_bytes, const float *x,
                 const float *router_weight, float *y, const MoeExtras *extras = nullptr,
                 HandleMemo *memo = nullptr);

/** the same block on device copies the caller already holds (experts entries each) */
void moe_forward_resident(const MoeShape &shape, const hipq_weight_t *gate, const hipq_weight_t *up,
                          const hipq_weight_t *down, const float *x, const float *router_weight, float *y,
                          const MoeExtras *extras = nullptr);

} // namespace hipq_host

#endif /* HIPQ_HOST_H */
