// SPDX-License-Identifier: Apache-2.0
/**
 * @file   fc_layer_hip.h
 * @brief  Fully connected layer whose quantized matmul runs on the GPU.
 *
 * Counterpart of FullyConnectedLayer (nntrainer/layers/fc_layer.cpp:51-304) and
 * of its OpenCL twin (nntrainer/layers/cl_layers/fc_layer_cl.cpp:37-163) for
 * weights of type Q4_0, Q4_K and Q6_K with fp32 activations: the inference path
 * of the quantized LLM applications. Same type string, same properties it
 * needs (unit, disable_bias), same tensors requested in finalize, same
 * forwarding / incremental_forwarding semantics.
 */
#ifndef HIPQ_FC_LAYER_HIP_H
#define HIPQ_FC_LAYER_HIP_H

#include <array>
#include <string>
#include <vector>

#include "nntr_api.h"

namespace nntrainer {

class FullyConnectedLayerHip : public Layer {
public:
  FullyConnectedLayerHip() = default;
  ~FullyConnectedLayerHip() override = default;

  void finalize(InitLayerContext &context) override;
  void forwarding(RunLayerContext &context, bool training) override;
  void incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                              bool training) override;
  /** inference only: there is no gradient of a block-quantized weight */
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
  const std::string getType() const override { return FullyConnectedLayerHip::type; }
  bool supportBackwarding() const override { return false; }

  inline static const std::string type = "fully_connected";

private:
  enum FCParams { weight, bias };

  /** output[M x unit] = input[M x K] . weight on the GPU, rows contiguous */
  void dotHip(const Tensor &input, const Tensor &weight, Tensor &output) const;

  unsigned int unit = 0;
  bool disable_bias = false;
  std::array<unsigned int, 2> weight_idx = {0, 0};
};

} // namespace nntrainer

#endif /* HIPQ_FC_LAYER_HIP_H */
