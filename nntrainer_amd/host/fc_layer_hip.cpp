// SPDX-License-Identifier: Apache-2.0
/**
 * @file   fc_layer_hip.cpp
 * @brief  FullyConnectedLayerHip (see fc_layer_hip.h).
 */
#include "fc_layer_hip.h"

#include "layer_common.h"
#include "layer_props.h"

namespace nntrainer {

static constexpr unsigned int SINGLE_INOUT_IDX = 0;

void FullyConnectedLayerHip::setProperty(const std::vector<std::string> &values) {
  for (const auto &kv : hipq_host::split_properties(values)) {
    const std::string &key = kv.first, &val = kv.second;
    if (key == "unit") {
      unit = hipq_host::parse_positive(key, val);
    } else if (key == "disable_bias") {
      disable_bias = hipq_host::parse_bool(key, val);
    } else if (key == "weight_initializer" || key == "bias_initializer" ||
               key == "weight_regularizer" || key == "weight_regularizer_constant" ||
               key == "weight_decay" || key == "bias_decay" || key == "print") {
      /* training-time properties of the CPU layer: accepted, without effect on inference */
    } else if (key == "lora_rank" || key == "lora_alpha") {
      throw exception::not_supported("FullyConnectedLayerHip does not run LoRA adapters");
    } else {
      throw std::invalid_argument("Unknown Layer Properties count 1: " + key);
    }
  }
}

void FullyConnectedLayerHip::finalize(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument)
    << "Fully connected layer takes only one input";
  NNTR_THROW_IF(unit == 0, std::invalid_argument) << "Fully connected layer needs the unit property";
  NNTR_THROW_IF(context.getFormat() != Tformat::NCHW, exception::not_supported)
    << "FullyConnectedLayerHip supports the NCHW format only";
  NNTR_THROW_IF(context.getActivationDataType() != Tdatatype::FP32, exception::not_supported)
    << "FullyConnectedLayerHip computes with fp32 activations";
  const Tdatatype wtype = context.getWeightDataType();
  NNTR_THROW_IF(hipq_dtype_of(wtype) < 0, exception::not_supported)
    << "FullyConnectedLayerHip serves Q4_0, Q4_K and Q6_K weights";

  std::vector<TensorDim> output_dims(1);

  /// @note same flags as the CPU layer: batch and width are effective, batch is dynamic
  context.setEffDimFlagInputDimension(0, 0b1001);
  context.setDynDimFlagInputDimension(0, 0b1000);

  auto const &in_dim = context.getInputDimensions()[0];
  const unsigned int block = wtype == Tdatatype::Q4_0 ? 32 : 256;
  NNTR_THROW_IF(in_dim.width() % block != 0, std::invalid_argument)
    << "input width " << in_dim.width() << " is not a multiple of the quantization block " << block;

  output_dims[0] = in_dim;
  output_dims[0].width(unit);
  output_dims[0].setTensorType({context.getFormat(), context.getActivationDataType()});
  context.setOutputDimensions(output_dims);

  /** Bias Dimension : (1, 1, 1, unit), activation type as in fc_layer.cpp:106-111 */
  TensorDim bias_dim(1, 1, 1, unit,
                     TensorDim::TensorType(context.getFormat(), context.getActivationDataType()), 0b0001);
  /** Weight Dimension : (1, 1, in_dim.width(), unit) */
  TensorDim weight_dim(1, 1, in_dim.width(), unit,
                       TensorDim::TensorType(context.getFormat(), context.getWeightDataType()), 0b0011);

  weight_idx[FCParams::weight] = context.requestWeight(
    weight_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f, "weight", true);
  if (!disable_bias)
    weight_idx[FCParams::bias] = context.requestWeight(
      bias_dim, Initializer::ZEROS, WeightRegularizer::NONE, 1.0f, 0.0f, "bias", true);
}

void FullyConnectedLayerHip::dotHip(const Tensor &input, const Tensor &weight, Tensor &output) const {
  /* as FloatTensor::dotQnK: M = height, K = width of the activation view,
   * N = width of the weight (float_tensor.cpp:935-940) */
  const int64_t M = (int64_t)input.batch() * input.channel() * input.height();
  const int64_t K = input.width();
  const int64_t N = weight.width();
  NNTR_THROW_IF((int64_t)weight.height() != K, std::invalid_argument)
    << "weight height " << weight.height() << " does not match input width " << K;
  NNTR_THROW_IF((int64_t)output.width() != N, std::invalid_argument)
    << "output width " << output.width() << " does not match unit " << N;
  const int dtype = hipq_dtype_of(weight.getDataType());
  NNTR_THROW_IF(dtype < 0, std::invalid_argument) << "Error: unsupported datatype";
  const hipq_host::WeightSpec spec{dtype, hipq_host::framework_layout(dtype), N, K};
  hipq_host::matmul(hipq_host::global_cache(), weight.getData<uint8_t>(), spec, input.getData<float>(),
                    M, K, output.getData<float>(), N);
}

void FullyConnectedLayerHip::forwarding(RunLayerContext &context, bool training) {
  NNTR_THROW_IF(training, exception::not_supported)
    << "FullyConnectedLayerHip is an inference layer";
  Tensor &weight = context.getWeight(weight_idx[FCParams::weight]);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);

  dotHip(input_, weight, hidden_);

  if (!disable_bias) {
    Tensor &bias = context.getWeight(weight_idx[FCParams::bias]);
    hidden_.add_i(bias);
  }
}

void FullyConnectedLayerHip::incremental_forwarding(RunLayerContext &context, unsigned int from,
                                                    unsigned int to, bool training) {
  NNTR_THROW_IF(training, exception::not_supported)
    << "FullyConnectedLayerHip is an inference layer";
  NNTR_THROW_IF(to <= from, std::invalid_argument)
    << "incremental step [" << from << ", " << to << ") is empty";
  Tensor &weight = context.getWeight(weight_idx[FCParams::weight]);
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);

  TensorDim input_dim = input_.getDim();
  TensorDim hidden_dim = hidden_.getDim();
  NNTR_THROW_IF(to - from > input_dim.height(), std::invalid_argument)
    << "incremental step of " << (to - from) << " rows exceeds the input height " << input_dim.height();

  TensorDim input_step_dim = input_dim;
  TensorDim hidden_step_dim = hidden_dim;
  input_step_dim.batch(1);
  input_step_dim.height(to - from);
  hidden_step_dim.batch(1);
  hidden_step_dim.height(to - from);

  /* Rows [0, to - from) of every batch entry, as fc_layer.cpp:266-296. The reference takes
   * the INPUT of entry b at b times the feature length of the OUTPUT (fc_layer.cpp:268-270);
   * for batch 1, every LLM call, that is offset 0 either way. The same rule here, so that a
   * graph that runs on both engines sees the same numbers; where it would leave the input
   * tensor (the reference then reads past its end) the call is refused instead. */
  /* A decode step of a batch: one row per entry, the entries hidden_dim.getFeatureLen() apart on
   * both sides. The reference multiplies them one by one (each an M = 1 product); the same
   * products go out as ONE call that keeps each row's bits (hipq_matmul_each_row): one pass over
   * the weights and one transfer each way instead of one per entry. */
  const size_t stride = hidden_dim.getFeatureLen();
  if (to - from == 1 && hidden_.batch() > 1 && stride >= input_dim.width() && stride >= hidden_dim.width() &&
      (size_t)(hidden_.batch() - 1) * stride + input_dim.width() <= input_.size()) {
    const int64_t K = input_dim.width(), N = weight.width();
    NNTR_THROW_IF((int64_t)weight.height() != K, std::invalid_argument)
      << "weight height " << weight.height() << " does not match input width " << K;
    NNTR_THROW_IF((int64_t)hidden_dim.width() != N, std::invalid_argument)
      << "output width " << hidden_dim.width() << " does not match unit " << N;
    const int dtype = hipq_dtype_of(weight.getDataType());
    NNTR_THROW_IF(dtype < 0, std::invalid_argument) << "Error: unsupported datatype";
    const hipq_host::WeightSpec spec{dtype, hipq_host::framework_layout(dtype), N, K};
    hipq_host::matmul_each_row(hipq_host::global_cache(), weight.getData<uint8_t>(), spec, input_.getData<float>(),
                               hidden_.batch(), (int64_t)stride, hidden_.getData<float>(), (int64_t)stride);
    if (!disable_bias) {
      Tensor &bias = context.getWeight(weight_idx[FCParams::bias]);
      for (unsigned int b = 0; b < hidden_.batch(); ++b) {
        Tensor hidden_step = hidden_.getSharedDataTensor(hidden_step_dim, b * stride, true);
        hidden_step.add_i(bias);
      }
    }
    return;
  }
  for (unsigned int b = 0; b < hidden_.batch(); ++b) {
    const size_t in_off = (size_t)b * hidden_dim.getFeatureLen();
    NNTR_THROW_IF(in_off + (size_t)(to - from) * input_dim.width() > input_.size(), std::invalid_argument)
      << "incremental_forwarding: batch entry " << b << " of the input lies outside the tensor";
    Tensor input_step = input_.getSharedDataTensor(input_step_dim, in_off, true);
    Tensor hidden_step =
      hidden_.getSharedDataTensor(hidden_step_dim, b * hidden_dim.getFeatureLen(), true);

    dotHip(input_step, weight, hidden_step);

    if (!disable_bias) {
      Tensor &bias = context.getWeight(weight_idx[FCParams::bias]);
      hidden_step.add_i(bias);
    }
  }
}

void FullyConnectedLayerHip::calcDerivative(RunLayerContext &) {
  throw exception::not_supported("FullyConnectedLayerHip does not support backwarding");
}

void FullyConnectedLayerHip::calcGradient(RunLayerContext &) {
  throw exception::not_supported("FullyConnectedLayerHip does not support backwarding");
}

void FullyConnectedLayerHip::read(std::ifstream &file, RunLayerContext &run_context, bool opt_var,
                   ml::train::ExecutionMode mode, bool trainable, TensorDim::DataType defineWeightDataType,
                   bool fsu, size_t start_offset, bool read_from_offset, int file_fd) {
  Layer::read(file, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset, file_fd);
  drop_device_copies(run_context);
}

void FullyConnectedLayerHip::read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
                   bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                   bool read_from_offset) {
  Layer::read(src, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset);
  drop_device_copies(run_context);
}

} // namespace nntrainer
