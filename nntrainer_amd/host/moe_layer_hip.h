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
 */
#ifndef HIPQ_MOE_LAYER_HIP_H
#define HIPQ_MOE_LAYER_HIP_H

#include <string>
#include <vector>

#include "nntr_api.h"

namespace nntrainer {

class MoELayerHip : public Layer {
public:
  MoELayerHip() = default;
  ~MoELayerHip() override = default;

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

private:
  /** the block on `tokens` rows of x -> y (both [tokens x hidden], contiguous) */
  void run(RunLayerContext &context, const float *x, float *y, unsigned int tokens,
           bool renormalize) const;

  unsigned int num_experts = 0;
  unsigned int topk = 0;
  unsigned int intermediate = 0;
  unsigned int hidden = 0;
  bool activation_set = false;
  int weight_dtype = -1;

  unsigned int gate_idx = 0;
  std::vector<unsigned int> expert_gate_proj_indices;
  std::vector<unsigned int> expert_up_proj_indices;
  std::vector<unsigned int> expert_down_proj_indices;
  unsigned int router_logits_idx = 0;
  unsigned int expert_mask_idx = 0;
};

} // namespace nntrainer

#endif /* HIPQ_MOE_LAYER_HIP_H */
