// SPDX-License-Identifier: Apache-2.0
/**
 * @file   mlp_swiglu_layer_hip.cpp
 * @brief  MlpSwiGLULayerHip (see mlp_swiglu_layer_hip.h).
 */
#include "mlp_swiglu_layer_hip.h"

#include "layer_common.h"
#include "layer_props.h"

namespace nntrainer {

static constexpr unsigned int SINGLE_INOUT_IDX = 0;

void MlpSwiGLULayerHip::setProperty(const std::vector<std::string> &values) {
  for (const auto &kv : hipq_host::split_properties(values)) {
    const std::string &key = kv.first, &val = kv.second;
    if (key == "unit") {
      unit = hipq_host::parse_positive(key, val);
    } else if (key == "down_unit") {
      down_unit = hipq_host::parse_positive(key, val);
    } else if (key == "disable_bias") {
      NNTR_THROW_IF(!hipq_host::parse_bool(key, val), exception::not_supported)
        << "MlpSwiGLULayerHip has no bias (the application's MLP FCs disable it, causal_lm.cpp:675-686)";
    } else if (key == "weight_initializer" || key == "weight_regularizer" ||
               key == "weight_regularizer_constant" || key == "weight_decay" || key == "print") {
      /* training-time properties: accepted, without effect on inference */
    } else {
      throw std::invalid_argument("Unknown Layer Properties count 1: " + key);
    }
  }
}

void MlpSwiGLULayerHip::finalize(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument) << "the gated MLP takes only one input";
  NNTR_THROW_IF(unit == 0, std::invalid_argument) << "the gated MLP needs the unit property";
  NNTR_THROW_IF(context.getFormat() != Tformat::NCHW, exception::not_supported)
    << "MlpSwiGLULayerHip supports the NCHW format only";
  NNTR_THROW_IF(context.getActivationDataType() != Tdatatype::FP32, exception::not_supported)
    << "MlpSwiGLULayerHip computes with fp32 activations";
  const Tdatatype wtype = context.getWeightDataType();
  NNTR_THROW_IF(hipq_dtype_of(wtype) < 0, exception::not_supported)
    << "MlpSwiGLULayerHip serves Q4_0, Q4_K and Q6_K weights";

  context.setEffDimFlagInputDimension(0, 0b1001);
  context.setDynDimFlagInputDimension(0, 0b1000);

  auto const &in_dim = context.getInputDimensions()[0];
  const unsigned int block = wtype == Tdatatype::Q4_0 ? 32 : 256;
  NNTR_THROW_IF(in_dim.width() % block != 0, std::invalid_argument)
    << "input width " << in_dim.width() << " is not a multiple of the quantization block " << block;

  NNTR_THROW_IF(down_unit && unit % block != 0, std::invalid_argument)
    << "unit " << unit << " is not a multiple of the quantization block " << block
    << " (the rows the down projection takes)";

  std::vector<TensorDim> output_dims(1);
  output_dims[0] = in_dim;
  output_dims[0].width(down_unit ? down_unit : unit);
  output_dims[0].setTensorType({context.getFormat(), context.getActivationDataType()});
  context.setOutputDimensions(output_dims);

  TensorDim weight_dim(1, 1, in_dim.width(), unit,
                       TensorDim::TensorType(context.getFormat(), context.getWeightDataType()), 0b0011);
  weight_idx[Params::up] = context.requestWeight(weight_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f,
                                                 "up_weight", true);
  weight_idx[Params::gate] = context.requestWeight(weight_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f,
                                                   0.0f, "gate_weight", true);
  if (down_unit) {
    TensorDim down_dim(1, 1, unit, down_unit,
                       TensorDim::TensorType(context.getFormat(), context.getWeightDataType()), 0b0011);
    weight_idx[Params::down] = context.requestWeight(down_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f,
                                                     0.0f, "down_weight", true);
  }
}

void MlpSwiGLULayerHip::run(RunLayerContext &context, const float *x, float *y, unsigned int rows) const {
  const Tensor &wu = context.getWeight(weight_idx[Params::up]);
  const Tensor &wg = context.getWeight(weight_idx[Params::gate]);
  const int dtype = hipq_dtype_of(wu.getDataType());
  NNTR_THROW_IF(dtype < 0, std::invalid_argument) << "Error: unsupported datatype";
  const int64_t K = wu.height(), N = wu.width();
  const hipq_host::WeightSpec spec{dtype, hipq_host::framework_layout(dtype), N, K};
  if (down_unit) {
    const Tensor &wd = context.getWeight(weight_idx[Params::down]);
    const hipq_host::WeightSpec dspec{dtype, hipq_host::framework_layout(dtype), (int64_t)wd.width(),
                                      (int64_t)wd.height()};
    hipq_host::mlp_swiglu_down(hipq_host::global_cache(), wu.getData<uint8_t>(), wg.getData<uint8_t>(), spec,
                               wd.getData<uint8_t>(), dspec, x, rows, K, y, dspec.N);
    return;
  }
  hipq_host::mlp_swiglu(hipq_host::global_cache(), wu.getData<uint8_t>(), wg.getData<uint8_t>(), spec, x, rows, K, y,
                        N);
}

void MlpSwiGLULayerHip::forwarding(RunLayerContext &context, bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "MlpSwiGLULayerHip is an inference layer";
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);
  run(context, input_.getData<float>(), hidden_.getData<float>(),
      (unsigned int)(input_.batch() * input_.channel() * input_.height()));
}

void MlpSwiGLULayerHip::incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                                               bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "MlpSwiGLULayerHip is an inference layer";
  NNTR_THROW_IF(to <= from, std::invalid_argument)
    << "incremental step [" << from << ", " << to << ") is empty";
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);
  NNTR_THROW_IF(to - from > input_.height(), std::invalid_argument)
    << "incremental step of " << (to - from) << " rows exceeds the input height " << input_.height();
  /* rows [0, to - from) of every batch entry, each entry at its own offset on both sides (what the
   * SwiGLU layer does with its inputs, swiglu.cpp:52-60) */
  for (unsigned int b = 0; b < input_.batch(); ++b)
    run(context, input_.getData<float>() + (size_t)b * input_.getDim().getFeatureLen(),
        hidden_.getData<float>() + (size_t)b * hidden_.getDim().getFeatureLen(), to - from);
}

void MlpSwiGLULayerHip::calcDerivative(RunLayerContext &) {
  throw exception::not_supported("MlpSwiGLULayerHip does not support backwarding");
}

void MlpSwiGLULayerHip::calcGradient(RunLayerContext &) {
  throw exception::not_supported("MlpSwiGLULayerHip does not support backwarding");
}

void MlpSwiGLULayerHip::read(std::ifstream &file, RunLayerContext &run_context, bool opt_var,
                             ml::train::ExecutionMode mode, bool trainable, TensorDim::DataType defineWeightDataType,
                             bool fsu, size_t start_offset, bool read_from_offset, int file_fd) {
  Layer::read(file, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset, file_fd);
  drop_device_copies(run_context);
}

void MlpSwiGLULayerHip::read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
                             bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                             bool read_from_offset) {
  Layer::read(src, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset);
  drop_device_copies(run_context);
}

} // namespace nntrainer
