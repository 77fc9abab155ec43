// SPDX-License-Identifier: Apache-2.0
/**
 * @file   moe_layer_hip.cpp
 * @brief  MoELayerHip (see moe_layer_hip.h).
 */
#include "moe_layer_hip.h"

#include <cstring>

#include "layer_common.h"
#include "layer_props.h"

namespace nntrainer {

static constexpr unsigned int SINGLE_INOUT_IDX = 0;

MoELayerHip::~MoELayerHip() {
  for (hipq_weight_t w : resident)
    hipq_host::release(w);
  drop_device_biases();
}

void MoELayerHip::setProperty(const std::vector<std::string> &values) {
  for (const auto &kv : hipq_host::split_properties(values)) {
    const std::string &key = kv.first, &val = kv.second;
    if (key == "num_experts") {
      num_experts = hipq_host::parse_positive(key, val);
    } else if (key == "num_experts_per_token") {
      topk = hipq_host::parse_positive(key, val);
    } else if (key == "unit") {
      intermediate = hipq_host::parse_positive(key, val);
    } else if (key == "moe_activation") {
      /* the expert MLP is SwiGLU: silu(gate) * up (qwen_moe_layer.cpp:357-372) */
      const std::string a = hipq_host::lower(val);
      if (a != "swish" && a != "silu")
        throw exception::not_supported("MoELayerHip computes the swish activation only, got " + val);
      activation_set = true;
    } else if (key == "weight_initializer" || key == "weight_regularizer" ||
               key == "weight_regularizer_constant" || key == "weight_decay" || key == "print" ||
               key == "disable_bias" || key == "bias_initializer" || key == "bias_decay") {
      /* training-time properties of the CPU layer: accepted, without effect on inference */
    } else {
      throw std::invalid_argument("Unknown Layer Properties count 1: " + key);
    }
  }
}

void MoELayerHip::finalize(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument)
    << "MoE layer only supports single input";
  NNTR_THROW_IF(num_experts == 0 || topk == 0 || intermediate == 0, std::invalid_argument)
    << "MoE layer needs num_experts, num_experts_per_token and unit";
  NNTR_THROW_IF(topk > num_experts, std::invalid_argument)
    << "num_experts_per_token " << topk << " exceeds num_experts " << num_experts;
  if (!activation_set)
    throw std::runtime_error("Activation type is not set for MoE layer");
  if (context.getActivationDataType() != Tdatatype::FP32)
    throw std::runtime_error("Unsupported activation data type for MoE layer");
  NNTR_THROW_IF(context.getFormat() != Tformat::NCHW, exception::not_supported)
    << "MoELayerHip supports the NCHW format only";

  switch (context.getWeightDataType()) {
  case Tdatatype::Q4_0:
    weight_dtype = HIPQ_Q4_0;
    break;
  case Tdatatype::Q4_K:
    weight_dtype = HIPQ_Q4_K;
    break;
  case Tdatatype::Q6_K:
    weight_dtype = HIPQ_Q6_K;
    break;
  default:
    throw exception::not_supported("MoELayerHip serves Q4_0, Q4_K and Q6_K expert weights");
  }

  const auto &in_dim = context.getInputDimensions()[SINGLE_INOUT_IDX];
  std::vector<TensorDim> output_dims(1);
  output_dims[SINGLE_INOUT_IDX] = in_dim;
  context.setOutputDimensions(output_dims);

  hidden = in_dim.width();
  const unsigned int block = weight_dtype == HIPQ_Q4_0 ? 32 : 256;
  NNTR_THROW_IF(hidden % block != 0 || intermediate % block != 0, std::invalid_argument)
    << "hidden " << hidden << " and unit " << intermediate << " must be multiples of the quantization block "
    << block;

  /* 1. router weight, always fp32 (and its bias: gpt_oss_moe_layer.cpp:94-101) */
  TensorDim gate_dim(1, 1, hidden, num_experts,
                     TensorDim::TensorType(context.getFormat(), Tdatatype::FP32), 0b0011);
  gate_idx = context.requestWeight(gate_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f,
                                   "gate", true);
  if (gpt_oss) {
    TensorDim gate_bias_dim(1, 1, 1, num_experts,
                            TensorDim::TensorType(context.getFormat(), context.getActivationDataType()));
    gate_bias_idx = context.requestWeight(gate_bias_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f,
                                          "gate_bias", false);
  }

  /* 2. experts, in the order the model file stores them: up, gate, down */
  expert_gate_proj_indices.clear();
  expert_up_proj_indices.clear();
  expert_down_proj_indices.clear();
  expert_gate_proj_indices.reserve(num_experts);
  expert_up_proj_indices.reserve(num_experts);
  expert_down_proj_indices.reserve(num_experts);

  TensorDim expert_gate_dim(1, 1, hidden, intermediate,
                            TensorDim::TensorType(context.getFormat(), context.getWeightDataType()),
                            0b0011);
  TensorDim expert_down_dim(1, 1, intermediate, hidden,
                            TensorDim::TensorType(context.getFormat(), context.getWeightDataType()),
                            0b0011);
  /* the cached layers request their expert tensors as virtual ones
   * (qwen_moe_layer_cached.cpp:134-152, gpt_oss_moe_layer_cached.cpp:140-173); the gpt_oss
   * layers put each projection's bias right behind it (gpt_oss_moe_layer.cpp:136-169) */
  expert_gate_bias_indices.clear();
  expert_up_bias_indices.clear();
  expert_down_bias_indices.clear();
  const TensorDim::TensorType act_type(context.getFormat(), context.getActivationDataType());
  TensorDim expert_gate_bias_dim(1, 1, 1, intermediate, act_type, 0b0011);
  TensorDim expert_down_bias_dim(1, 1, 1, hidden, act_type, 0b0011);
  auto request = [&](const TensorDim &dim, const std::string &name) {
    return context.requestWeight(dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f, name, false,
                                 cached);
  };
  for (unsigned int i = 0; i < num_experts; ++i) {
    const std::string n = std::to_string(i);
    expert_up_proj_indices.push_back(request(expert_gate_dim, "expert_up_" + n));
    if (gpt_oss)
      expert_up_bias_indices.push_back(request(expert_gate_bias_dim, "expert_up_bias_" + n));
    expert_gate_proj_indices.push_back(request(expert_gate_dim, "expert_gate_" + n));
    if (gpt_oss)
      expert_gate_bias_indices.push_back(request(expert_gate_bias_dim, "expert_gate_bias_" + n));
    expert_down_proj_indices.push_back(request(expert_down_dim, "expert_down_" + n));
    if (gpt_oss)
      expert_down_bias_indices.push_back(request(expert_down_bias_dim, "expert_down_bias_" + n));
  }

  /* 3. the scratch tensors of the CPU layer, kept so that tensor indices and
   *    memory planning of a model do not depend on the engine */
  const unsigned int total_tokens = in_dim.batch() * in_dim.height();
  router_logits_idx =
    context.requestTensor({total_tokens, 1, 1, num_experts}, "router_logits", Initializer::NONE, false,
                          TensorLifespan::FORWARD_FUNC_LIFESPAN);
  expert_mask_idx =
    context.requestTensor({num_experts, 1, topk, total_tokens}, "expert_mask", Initializer::ZEROS,
                          false, TensorLifespan::FORWARD_FUNC_LIFESPAN);
}

void MoELayerHip::run(RunLayerContext &context, const float *x, float *y, unsigned int tokens,
                      bool renormalize, bool with_router_bias) {
  const unsigned int E = num_experts;
  hipq_host::MoeShape shape;
  shape.tokens = (int)tokens;
  shape.hidden = (int)hidden;
  shape.intermediate = (int)intermediate;
  shape.experts = (int)E;
  shape.topk = (int)topk;
  shape.renormalize = renormalize;
  /* the router weight stays on the device between steps (1 MB at 2048 x 128) */
  const float *router = dev_router.get(context.getWeight(gate_idx).getData<float>(), (size_t)hidden * E);

  /* a virtual tensor has bytes only between activate() and deactivate() */
  auto with_bytes = [&](unsigned int idx, auto use) {
    Tensor &t = context.getWeight(idx);
    if (cached)
      t.activate();
    use(t);
    if (cached)
      t.deactivate();
  };

  hipq_host::MoeExtras extras;
  extras.router_on_device = true;
  if (gpt_oss) {
    /* the biases go to the device once, with the weights: [E x I], [E x I], [E x H] gathered from
     * the experts' tensors, and the router's [E]; read() drops them as it drops the weights */
    if (!dev_bias_gate) {
      std::vector<float> bias_gate((size_t)E * intermediate), bias_up((size_t)E * intermediate),
        bias_down((size_t)E * hidden);
      for (unsigned int e = 0; e < E; ++e) {
        with_bytes(expert_gate_bias_indices[e], [&](Tensor &t) {
          std::memcpy(&bias_gate[(size_t)e * intermediate], t.getData<float>(), (size_t)intermediate * 4);
        });
        with_bytes(expert_up_bias_indices[e], [&](Tensor &t) {
          std::memcpy(&bias_up[(size_t)e * intermediate], t.getData<float>(), (size_t)intermediate * 4);
        });
        with_bytes(expert_down_bias_indices[e], [&](Tensor &t) {
          std::memcpy(&bias_down[(size_t)e * hidden], t.getData<float>(), (size_t)hidden * 4);
        });
      }
      dev_bias_gate = hipq_host::device_floats(bias_gate.data(), bias_gate.size());
      dev_bias_up = hipq_host::device_floats(bias_up.data(), bias_up.size());
      dev_bias_down = hipq_host::device_floats(bias_down.data(), bias_down.size());
    }
    if (with_router_bias && !dev_bias_router)
      dev_bias_router = hipq_host::device_floats(context.getWeight(gate_bias_idx).getData<float>(), E);
    extras.gpt_oss = true;
    extras.alpha = 1.702f; /* gpt_oss_moe_layer.h:126 */
    /* only the cached layer clamps (gpt_oss_moe_layer_cached.cpp:497-507, limit 7.0 from
     * gpt_oss_moe_layer_cached.h:137); the uncached one has the two lines commented out
     * (gpt_oss_moe_layer.cpp:414, 419) */
    extras.limit = cached ? 7.0f : 0.f;
    extras.gate_bias = dev_bias_gate;
    extras.up_bias = dev_bias_up;
    extras.down_bias = dev_bias_down;
    extras.router_bias = with_router_bias ? dev_bias_router : nullptr;
    extras.biases_on_device = true;
  }

  if (cached) {
    /* every expert once into HBM, where it stays: the reference's 32-entry LRU over host
     * memory (qwen_moe_layer_cached.cpp:376-454) has nothing to manage here */
    if (resident.empty()) {
      resident.assign(3 * (size_t)E, nullptr);
      const int layout = hipq_host::framework_layout(weight_dtype);
      const hipq_host::WeightSpec gu{weight_dtype, layout, (int64_t)intermediate, (int64_t)hidden};
      const hipq_host::WeightSpec dn{weight_dtype, layout, (int64_t)hidden, (int64_t)intermediate};
      for (unsigned int e = 0; e < E; ++e) {
        with_bytes(expert_gate_proj_indices[e],
                   [&](Tensor &t) { resident[e] = hipq_host::upload(t.getData<uint8_t>(), gu); });
        with_bytes(expert_up_proj_indices[e],
                   [&](Tensor &t) { resident[E + e] = hipq_host::upload(t.getData<uint8_t>(), gu); });
        with_bytes(expert_down_proj_indices[e],
                   [&](Tensor &t) { resident[2 * (size_t)E + e] = hipq_host::upload(t.getData<uint8_t>(), dn); });
      }
    }
    hipq_host::moe_forward_resident(shape, resident.data(), resident.data() + E, resident.data() + 2 * (size_t)E,
                                    x, router, y, &extras);
    return;
  }

  std::vector<const void *> g(E), u(E), d(E);
  for (unsigned int e = 0; e < E; ++e) {
    g[e] = context.getWeight(expert_gate_proj_indices[e]).getData<uint8_t>();
    u[e] = context.getWeight(expert_up_proj_indices[e]).getData<uint8_t>();
    d[e] = context.getWeight(expert_down_proj_indices[e]).getData<uint8_t>();
  }
  hipq_host::moe_forward(hipq_host::global_cache(), shape, weight_dtype, g, u, d, x, router, y, &extras, &handles);
}

void MoELayerHip::forwarding(RunLayerContext &context, bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "MoELayerHip is an inference layer";
  if (cached) /* the cached layers run by steps only (qwen_moe_layer_cached.cpp:173-174) */
    return;
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &output_ = context.getOutput(SINGLE_INOUT_IDX);
  const unsigned int total_tokens = input_.batch() * input_.height();
  /* the whole-tensor path keeps the softmax weights as they are (qwen_moe_layer.cpp:161-259
   * does not renormalise) and, in the gpt_oss layer, leaves the router bias out
   * (gpt_oss_moe_layer.cpp:209-212) */
  run(context, input_.getData<float>(), output_.getData<float>(), total_tokens, false, false);
}

void MoELayerHip::incremental_forwarding(RunLayerContext &context, unsigned int from,
                                         unsigned int to, bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "MoELayerHip is an inference layer";
  NNTR_THROW_IF(to <= from, std::invalid_argument)
    << "incremental step [" << from << ", " << to << ") is empty";
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &output_ = context.getOutput(SINGLE_INOUT_IDX);
  NNTR_THROW_IF(to - from > input_.height(), std::invalid_argument)
    << "incremental step of " << (to - from) << " rows exceeds the input height " << input_.height();

  TensorDim input_step_dim = input_.getDim();
  TensorDim output_step_dim = output_.getDim();
  input_step_dim.batch(1);
  output_step_dim.batch(1);
  input_step_dim.height(to - from);
  output_step_dim.height(to - from);

  /* rows [0, to - from) of every batch entry, as qwen_moe_layer.cpp:417-424 */
  for (unsigned int b = 0; b < input_.batch(); ++b) {
    Tensor input =
      input_.getSharedDataTensor(input_step_dim, b * input_.getDim().getFeatureLen(), true);
    Tensor output =
      output_.getSharedDataTensor(output_step_dim, b * output_.getDim().getFeatureLen(), true);
    /* of the two gpt_oss layers only the uncached one adds the router bias
     * (gpt_oss_moe_layer.cpp:500-504 against gpt_oss_moe_layer_cached.cpp:243-246) */
    run(context, input.getData<float>(), output.getData<float>(), to - from, true, gpt_oss && !cached);
  }
}

void MoELayerHip::drop_device_biases() noexcept {
  hipq_host::device_release(dev_bias_gate);
  hipq_host::device_release(dev_bias_up);
  hipq_host::device_release(dev_bias_down);
  hipq_host::device_release(dev_bias_router);
  dev_bias_gate = dev_bias_up = dev_bias_down = dev_bias_router = nullptr;
  dev_router.drop();
}

void MoELayerHip::calcDerivative(RunLayerContext &) {
  throw exception::not_supported("MoELayerHip does not support backwarding");
}

void MoELayerHip::calcGradient(RunLayerContext &) {
  throw exception::not_supported("MoELayerHip does not support backwarding");
}

/* of a cached layer also the copies it holds itself: the next step uploads again */
#define HIPQ_MOE_DROP_RESIDENT()                                                                    \
  do {                                                                                              \
    for (hipq_weight_t w : resident)                                                                \
      hipq_host::release(w);                                                                        \
    resident.clear();                                                                               \
    drop_device_biases();                                                                           \
  } while (0)

void MoELayerHip::read(std::ifstream &file, RunLayerContext &run_context, bool opt_var,
                   ml::train::ExecutionMode mode, bool trainable, TensorDim::DataType defineWeightDataType,
                   bool fsu, size_t start_offset, bool read_from_offset, int file_fd) {
  Layer::read(file, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset, file_fd);
  drop_device_copies(run_context);
  HIPQ_MOE_DROP_RESIDENT();
}

void MoELayerHip::read(ReadSource src, RunLayerContext &run_context, bool opt_var, ml::train::ExecutionMode mode,
                   bool trainable, TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                   bool read_from_offset) {
  Layer::read(src, run_context, opt_var, mode, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset);
  drop_device_copies(run_context);
  HIPQ_MOE_DROP_RESIDENT();
}

} // namespace nntrainer
