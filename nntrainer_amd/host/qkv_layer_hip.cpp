// SPDX-License-Identifier: Apache-2.0
/**
 * @file   qkv_layer_hip.cpp
 * @brief  QKVLayerHip (see qkv_layer_hip.h).
 */
#include "qkv_layer_hip.h"

#include "layer_common.h"
#include "layer_props.h"

namespace nntrainer {

static constexpr unsigned int SINGLE_INOUT_IDX = 0;

void QKVLayerHip::setProperty(const std::vector<std::string> &values) {
  for (const auto &kv : hipq_host::split_properties(values)) {
    const std::string &key = kv.first, &val = kv.second;
    if (key == "q_unit") {
      unit[Q] = hipq_host::parse_positive(key, val);
    } else if (key == "k_unit") {
      unit[K] = hipq_host::parse_positive(key, val);
    } else if (key == "v_unit") {
      unit[V] = hipq_host::parse_positive(key, val);
    } else if (key == "weight_initializer" || key == "bias_initializer" || key == "weight_regularizer" ||
               key == "weight_regularizer_constant" || key == "weight_decay" || key == "bias_decay" ||
               key == "disable_bias" || key == "print") {
      /* LayerImpl's training-time properties: accepted, without effect on inference */
    } else {
      throw std::invalid_argument("Unknown Layer Properties count 1: " + key);
    }
  }
}

void QKVLayerHip::finalize(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument)
    << "Fully connected layer takes only one input";
  NNTR_THROW_IF(unit[Q] == 0 || unit[K] == 0 || unit[V] == 0, std::invalid_argument)
    << "QKV layer needs q_unit, k_unit and v_unit";
  NNTR_THROW_IF(context.getFormat() != Tformat::NCHW, exception::not_supported)
    << "QKVLayerHip supports the NCHW format only";
  NNTR_THROW_IF(context.getActivationDataType() != Tdatatype::FP32, exception::not_supported)
    << "QKVLayerHip computes with fp32 activations";
  const Tdatatype wtype = context.getWeightDataType();
  NNTR_THROW_IF(hipq_dtype_of(wtype) < 0, exception::not_supported)
    << "QKVLayerHip serves Q4_0, Q4_K and Q6_K weights";

  context.setEffDimFlagInputDimension(0, 0b1001);
  context.setDynDimFlagInputDimension(0, 0b1000);

  auto const &in_dim = context.getInputDimensions()[0];
  const unsigned int block = wtype == Tdatatype::Q4_0 ? 32 : 256;
  NNTR_THROW_IF(in_dim.width() % block != 0, std::invalid_argument)
    << "input width " << in_dim.width() << " is not a multiple of the quantization block " << block;

  std::vector<TensorDim> output_dims(3);
  for (int i = 0; i < 3; ++i) {
    output_dims[i] = in_dim;
    output_dims[i].width(unit[i]);
    output_dims[i].setTensorType({context.getFormat(), context.getActivationDataType()});
  }
  context.setOutputDimensions(output_dims);

  static const char *names[3] = {"qweight", "kweight", "vweight"};
  for (int i = 0; i < 3; ++i) {
    TensorDim weight_dim(1, 1, in_dim.width(), unit[i],
                         TensorDim::TensorType(context.getFormat(), context.getWeightDataType()), 0b0011);
    weight_idx[i] = context.requestWeight(weight_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f,
                                          names[i], true);
  }
}

void QKVLayerHip::forwarding(RunLayerContext &, bool) {}

void QKVLayerHip::incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                                         bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "QKVLayerHip is an inference layer";
  NNTR_THROW_IF(to <= from, std::invalid_argument)
    << "incremental step [" << from << ", " << to << ") is empty";
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  NNTR_THROW_IF(to - from > input_.height(), std::invalid_argument)
    << "incremental step of " << (to - from) << " rows exceeds the input height " << input_.height();

  /* rows [0, to - from) of the first batch entry on both sides, as qkv_layer.cpp:143-173 */
  const int64_t M = to - from;
  const int64_t K = input_.width();
  std::vector<const void *> bytes(3);
  std::vector<hipq_host::WeightSpec> specs(3);
  std::vector<float *> outs(3);
  for (int i = 0; i < 3; ++i) {
    const Tensor &w = context.getWeight(weight_idx[i]);
    NNTR_THROW_IF((int64_t)w.height() != K, std::invalid_argument)
      << "weight height " << w.height() << " does not match input width " << K;
    const int dtype = hipq_dtype_of(w.getDataType());
    NNTR_THROW_IF(dtype < 0, std::invalid_argument) << "Error: unsupported datatype";
    bytes[i] = w.getData<uint8_t>();
    specs[i] = hipq_host::WeightSpec{dtype, hipq_host::framework_layout(dtype), (int64_t)w.width(), K};
    Tensor &out = context.getOutput(i);
    NNTR_THROW_IF((int64_t)out.width() != (int64_t)w.width(), std::invalid_argument)
      << "output width " << out.width() << " does not match unit " << w.width();
    outs[i] = out.getData<float>();
  }
  hipq_host::matmul_multi(hipq_host::global_cache(), bytes, specs, input_.getData<float>(), M, K, outs);
}

void QKVLayerHip::calcDerivative(RunLayerContext &) {
  throw exception::not_supported("QKVLayerHip does not support backwarding");
}

void QKVLayerHip::calcGradient(RunLayerContext &) {
  throw exception::not_supported("QKVLayerHip does not support backwarding");
}

void QKVLayerHip::read(std::ifstream &file, RunLayerContext &run_context, bool opt_var,
                       ml::train::ExecutionMode mode, bool trainable, TensorDim::DataType defineWeightDataType,
                       bool fsu, size_t start_offset, bool read_from_offset, int file_fd) {
  Layer::read(file, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset, file_fd);
  drop_device_copies(run_context);
}

void QKVLayerHip::read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
                       bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                       bool read_from_offset) {
  Layer::read(src, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset);
  drop_device_copies(run_context);
}

} // namespace nntrainer
