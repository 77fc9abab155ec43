// SPDX-License-Identifier: Apache-2.0
/**
 * @file   qkv_layer_hip.h
 * @brief  The Q, K and V projections of an attention block as one layer whose three
 *         quantized products share one activation quantization on the GPU.
 *
 * Counterpart of causallm::QKVLayer (Applications/CausalLM/layers/qkv_layer.cpp:43-110
 * finalize, 132-181 incremental_forwarding; type key "qkv_layer", qkv_layer.h:143;
 * properties q_unit, k_unit, v_unit, qkv_layer.h:33-58). It requests the same three
 * weights in the same order ("qweight", "kweight", "vweight", [in_width x unit] of the model's
 * weight type) and produces the same three outputs, so a graph built by
 * nntr_qwen3_causallm.cpp:46-56 and a model file written for the CPU layer work unchanged.
 * The reference hands the three weights to Tensor::dot(vector) (float_tensor.cpp:724-798),
 * which quantizes the activation once; so does hipq_matmul_multi, and for one row it is a
 * single kernel launch for all three.
 */
#ifndef HIPQ_QKV_LAYER_HIP_H
#define HIPQ_QKV_LAYER_HIP_H

#include <array>
#include <string>
#include <vector>

#include "nntr_api.h"

namespace nntrainer {

class QKVLayerHip : public Layer {
public:
  QKVLayerHip() = default;
  ~QKVLayerHip() override = default;

  void finalize(InitLayerContext &context) override;
  /** a no-op, as in the reference (qkv_layer.cpp:128-130): the layer runs by steps */
  void forwarding(RunLayerContext &context, bool training) override;
  void incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                              bool training) override;
  void calcDerivative(RunLayerContext &context) override;
  void calcGradient(RunLayerContext &context) override;
  void setProperty(const std::vector<std::string> &values) override;
  /** see FullyConnectedLayerHip::read */
  void read(std::ifstream &file, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
            bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset = 0,
            bool read_from_offset = false, int file_fd = -1) override;
  void read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
            bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset = 0,
            bool read_from_offset = false) override;
  const std::string getType() const override { return QKVLayerHip::type; }
  bool supportBackwarding() const override { return false; }

  inline static const std::string type = "qkv_layer";

private:
  enum QKVParams { Q, K, V };
  std::array<unsigned int, 3> unit = {0, 0, 0};
  std::array<unsigned int, 3> weight_idx = {0, 0, 0};
};

} // namespace nntrainer

#endif /* HIPQ_QKV_LAYER_HIP_H */
