// SPDX-License-Identifier: Apache-2.0
/**
 * @file   moe_layer_hip.h
 * @brief  Mixture-of-experts FFN block whose routing, token sort and expert
 *         MLPs run on the GPU in one grouped launch sequence.
 *
 * Counterpart of MoELayer (Applications/CausalLM/layers/qwen_moe_layer.cpp:50-159
 * finalize, 394-503 incremental_forwarding, 332-392 expert forward; type key
 * "qwen_moe", qwen_moe_layer.h:107; properties num_experts,
 * num_experts_per_token, unit, moe_activation,
 * causallm_common_properties.h:44-69). It requests the same weights in the same
 * order (router "gate" fp32 [H x E], then per expert up, gate, down in the model
 * weight type) so that a model file written for the CPU layer loads unchanged.
 *
 * The same class, configured by its constructor, stands in for the application's other three
 * MoE layers; each is registered under the reference's own type key:
 *  - "moe_cached_slim" (CachedSlimMoELayer, qwen_moe_layer_cached.cpp): the expert weights are
 *    virtual tensors the CPU layer maps in on demand and keeps 32 of (LRU, :376-454). Here an
 *    expert is activated once, stored in HBM, deactivated again and stays resident for the life
 *    of the layer: 288 GB of HBM hold every expert of the models this path serves, so there is
 *    nothing to evict. The batched product per expert (:176-265) is how every MoE runs here.
 *    forwarding() is a no-op as in the reference (:173-174).
 *  - "gpt_oss_moe" (GptOssMoELayer, gpt_oss_moe_layer.cpp): router bias, biased projections,
 *    h = (g / (1 + exp(-1.702 g))) * (u + 1), biased down projection (:372-449); the router bias
 *    enters in incremental_forwarding (:500-504) and not in forwarding (:209-212), as there.
 *  - "gpt_oss_moe_slim_cached" (CachedSlimGptOssMoELayer, gpt_oss_moe_layer_cached.cpp): the
 *    two together; this one never adds the router bias (:243-246), as there.
 */
#ifndef HIPQ_MOE_LAYER_HIP_H
#define HIPQ_MOE_LAYER_HIP_H

#include <string>
#include <vector>

#include <hipq.h>

#include "hipq_host.h"

#include "nntr_api.h"

namespace nntrainer {

class MoELayerHip : public Layer {
public:
  MoELayerHip() = default;
  ~MoELayerHip() override;

  void finalize(InitLayerContext &context) override;
  void forwarding(RunLayerContext &context, bool training) override;
  void incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                              bool training) override;
  void calcDerivative(RunLayerContext &context) override;
  void calcGradient(RunLayerContext &context) override;
  void setProperty(const std::vector<std::string> &values) override;
  /** The framework reads the weights into the tensors it owns; the device copies made from
   *  their earlier content (a first forward before the load, a reload, a buffer that a
   *  swapped-in weight shares) are dropped, so the next forward uploads the new bytes. */
  void read(std::ifstream &file, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
            bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset = 0,
            bool read_from_offset = false, int file_fd = -1) override;
  void read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
            bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset = 0,
            bool read_from_offset = false) override;
  const std::string getType() const override { return MoELayerHip::type; }
  bool supportBackwarding() const override { return false; }

  inline static const std::string type = "qwen_moe";

protected:
  /** gpt_oss: the biased variant; cached: virtual expert weights, resident copies */
  MoELayerHip(bool gpt_oss_, bool cached_) : gpt_oss(gpt_oss_), cached(cached_), activation_set(gpt_oss_) {}

private:
  /** the block on `tokens` rows of x -> y (both [tokens x hidden], contiguous) */
  void run(RunLayerContext &context, const float *x, float *y, unsigned int tokens, bool renormalize,
           bool with_router_bias);

  bool gpt_oss = false;
  bool cached = false;

  bool activation_set = false; /* the gpt_oss layers have no moe_activation property */
  unsigned int num_experts = 0;
  unsigned int topk = 0;
  unsigned int intermediate = 0;
  unsigned int hidden = 0;
  int weight_dtype = -1;

  unsigned int gate_idx = 0;
  std::vector<unsigned int> expert_gate_proj_indices;
  std::vector<unsigned int> expert_up_proj_indices;
  std::vector<unsigned int> expert_down_proj_indices;
  unsigned int router_logits_idx = 0;
  unsigned int expert_mask_idx = 0;
  /* gpt_oss */
  unsigned int gate_bias_idx = 0;
  std::vector<unsigned int> expert_gate_bias_indices;
  std::vector<unsigned int> expert_up_bias_indices;
  std::vector<unsigned int> expert_down_bias_indices;
  /* device copies of the biases, [E x I], [E x I], [E x H] and the router's [E]: made at the first
   * step, dropped when the framework reads the layer's weights again */
  float *dev_bias_gate = nullptr, *dev_bias_up = nullptr, *dev_bias_down = nullptr, *dev_bias_router = nullptr;
  void drop_device_biases() noexcept;
  hipq_host::DeviceMirror dev_router; /* the fp32 router weight [hidden x experts] */
  /* cached: device copies this layer owns, gate | up | down, made at an expert's first use */
  std::vector<hipq_weight_t> resident;
  hipq_host::HandleMemo handles; /* the uncached layers' expert handles from the last call */
};

/** "moe_cached_slim" */
class CachedSlimMoELayerHip : public MoELayerHip {
public:
  CachedSlimMoELayerHip() : MoELayerHip(false, true) {}
  const std::string getType() const override { return CachedSlimMoELayerHip::type; }
  inline static const std::string type = "moe_cached_slim";
};

/** "gpt_oss_moe" */
class GptOssMoELayerHip : public MoELayerHip {
public:
  GptOssMoELayerHip() : MoELayerHip(true, false) {}
  const std::string getType() const override { return GptOssMoELayerHip::type; }
  inline static const std::string type = "gpt_oss_moe";
};

/** "gpt_oss_moe_slim_cached" */
class CachedSlimGptOssMoELayerHip : public MoELayerHip {
public:
  CachedSlimGptOssMoELayerHip() : MoELayerHip(true, true) {}
  const std::string getType() const override { return CachedSlimGptOssMoELayerHip::type; }
  inline static const std::string type = "gpt_oss_moe_slim_cached";
};

} // namespace nntrainer

#endif /* HIPQ_MOE_LAYER_HIP_H */
