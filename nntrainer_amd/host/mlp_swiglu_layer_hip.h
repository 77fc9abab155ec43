// SPDX-License-Identifier: Apache-2.0
/**
 * @file   mlp_swiglu_layer_hip.h
 * @brief  The gated half of a dense MLP as one layer: out = swiglu(x . W_up, x . W_gate).
 *
 * The LLM application builds this from three layers (CausalLM::createMlp,
 * Applications/CausalLM/causal_lm.cpp:672-695): the FCs "ffn_up" and "ffn_gate" on the same
 * input and a SwiGLULayer on their outputs (layers/swiglu.cpp:40-62: swiglu(N, out, in0, in1)
 * with in0 = ffn_up, in1 = ffn_gate, i.e. out = (up / (1 + exp(-up))) * gate). On the GPU the
 * three are one call: the activation is quantized once and, for a decode step, the two products
 * and the SwiGLU are one kernel launch. There is no such layer in the framework; a graph that
 * wants it replaces the three createLayer calls with one of type "mlp_swiglu" (property `unit` =
 * the MLP's hidden size). It requests "up_weight" then "gate_weight", [in_width x unit] of the
 * model's weight type: the order in which the two FCs' weights lie in a model file, so files
 * written for the three-layer form load unchanged.
 *
 * With the property `down_unit` (the model's width) the layer is the whole MLP of createMlp
 * (causal_lm.cpp:671-705), the FC "ffn_down" included: it requests "down_weight" [unit x down_unit]
 * after the other two (again the file's order), its output is [rows x down_unit], and the hidden
 * rows never leave the device (hipq_mlp_swiglu_down): one call and one wait where the layers
 * "mlp_swiglu" + "fully_connected" move the hidden rows to the host and back.
 */
#ifndef HIPQ_MLP_SWIGLU_LAYER_HIP_H
#define HIPQ_MLP_SWIGLU_LAYER_HIP_H

#include <array>
#include <string>
#include <vector>

#include "nntr_api.h"

namespace nntrainer {

class MlpSwiGLULayerHip : public Layer {
public:
  MlpSwiGLULayerHip() = default;
  ~MlpSwiGLULayerHip() override = default;

  void finalize(InitLayerContext &context) override;
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
  const std::string getType() const override { return MlpSwiGLULayerHip::type; }
  bool supportBackwarding() const override { return false; }

  inline static const std::string type = "mlp_swiglu";

private:
  enum Params { up, gate, down };
  void run(RunLayerContext &context, const float *x, float *y, unsigned int rows) const;

  unsigned int unit = 0;
  unsigned int down_unit = 0; /* 0: the gated half only */
  std::array<unsigned int, 3> weight_idx = {0, 0, 0};
};

} // namespace nntrainer

#endif /* HIPQ_MLP_SWIGLU_LAYER_HIP_H */
