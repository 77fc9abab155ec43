// SPDX-License-Identifier: Apache-2.0
/**
 * @file   tie_word_embedding_hip.cpp
 * @brief  TieWordEmbeddingHip (see tie_word_embedding_hip.h).
 */
#include "tie_word_embedding_hip.h"

#include <cstring>

#include "layer_common.h"
#include "layer_props.h"

namespace nntrainer {

static constexpr unsigned int SINGLE_INOUT_IDX = 0;

void TieWordEmbeddingHip::setProperty(const std::vector<std::string> &values) {
  for (const auto &kv : hipq_host::split_properties(values)) {
    const std::string &key = kv.first, &val = kv.second;
    if (key == "in_dim") {
      in_dim = hipq_host::parse_positive(key, val);
    } else if (key == "out_dim") {
      out_dim = hipq_host::parse_positive(key, val);
    } else if (key == "unit") {
      unit = hipq_host::parse_positive(key, val);
    } else if (key == "disable_bias") {
      disable_bias = hipq_host::parse_bool(key, val);
    } else if (key == "weight_initializer" || key == "bias_initializer" || key == "weight_regularizer" ||
               key == "weight_regularizer_constant" || key == "weight_decay" || key == "bias_decay" ||
               key == "print") {
      /* LayerImpl's training-time properties: accepted, without effect on inference */
    } else {
      throw std::invalid_argument("Unknown Layer Properties count 1: " + key);
    }
  }
}

void TieWordEmbeddingHip::finalize(InitLayerContext &context) {
  mode = unit == 0 ? Mode::embedding : Mode::lm_head;
  if (mode == Mode::embedding)
    finalize_embedding(context);
  else
    finalize_lmhead(context);
}

void TieWordEmbeddingHip::finalize_embedding(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument) << "Embedding layer takes only one input";
  NNTR_THROW_IF(in_dim == 0 || out_dim == 0, std::invalid_argument) << "Embedding layer needs in_dim and out_dim";
  const TensorDim &input_dim = context.getInputDimensions()[SINGLE_INOUT_IDX];
  NNTR_THROW_IF(input_dim.channel() != 1, std::invalid_argument)
    << "Embedding layer takes only one for channel size";
  NNTR_THROW_IF(input_dim.getDataType() != Tdatatype::FP32, std::invalid_argument)
    << "Embedding layer takes only FP32 input data";
  const Tdatatype wtype = context.getWeightDataType();
  NNTR_THROW_IF(wtype != Tdatatype::Q6_K && wtype != Tdatatype::FP32, std::invalid_argument)
    << "Tieword embedding is not supported yet for the data type";
  NNTR_THROW_IF(wtype == Tdatatype::Q6_K && out_dim % 256 != 0, std::invalid_argument)
    << "out_dim " << out_dim << " is not a multiple of the quantization block 256";

  /* one output row per input id: [b, 1, ids, out_dim] */
  TensorDim output_dim = input_dim;
  output_dim.height(input_dim.width());
  output_dim.width(out_dim);
  output_dim.setTensorType({context.getFormat(), context.getActivationDataType()});
  context.setOutputDimensions({output_dim});

  TensorDim dim = output_dim;
  dim.setTensorType({context.getFormat(), context.getWeightDataType()});
  dim.height(in_dim);
  dim.width(out_dim);
  dim.batch(1);
  weight_idx[Params::weight] =
    context.requestWeight(dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f, "Embedding", true);
}

void TieWordEmbeddingHip::finalize_lmhead(InitLayerContext &context) {
  NNTR_THROW_IF(context.getNumInputs() != 1, std::invalid_argument) << "lm head layer takes only one input";
  NNTR_THROW_IF(context.getFormat() != Tformat::NCHW, exception::not_supported)
    << "TieWordEmbeddingHip supports the NCHW format only";
  NNTR_THROW_IF(context.getActivationDataType() != Tdatatype::FP32, exception::not_supported)
    << "TieWordEmbeddingHip computes with fp32 activations";
  const Tdatatype wtype = context.getWeightDataType();
  NNTR_THROW_IF(hipq_dtype_of(wtype) < 0, exception::not_supported)
    << "TieWordEmbeddingHip serves Q4_0, Q4_K and Q6_K weights as the lm_head";

  context.setEffDimFlagInputDimension(0, 0b1001);
  context.setDynDimFlagInputDimension(0, 0b1000);

  auto const &idim = context.getInputDimensions()[0];
  const unsigned int block = wtype == Tdatatype::Q4_0 ? 32 : 256;
  NNTR_THROW_IF(idim.width() % block != 0, std::invalid_argument)
    << "input width " << idim.width() << " is not a multiple of the quantization block " << block;

  std::vector<TensorDim> output_dims(1);
  output_dims[0] = idim;
  output_dims[0].width(unit);
  output_dims[0].setTensorType({context.getFormat(), context.getActivationDataType()});
  context.setOutputDimensions(output_dims);

  /* both of the weight type, as tie_word_embedding.cpp:137-151; the weight transposed so that it
   * is the embedding table: unit rows of in_width values */
  TensorDim bias_dim(1, 1, 1, unit, TensorDim::TensorType(context.getFormat(), context.getWeightDataType()),
                     0b0001);
  TensorDim weight_dim(1, 1, unit, idim.width(),
                       TensorDim::TensorType(context.getFormat(), context.getWeightDataType()), 0b0011);
  weight_idx[Params::weight] =
    context.requestWeight(weight_dim, Initializer::NONE, WeightRegularizer::NONE, 1.0f, 0.0f, "Embedding", true);
  /* the reference requests the bias in the weight's (quantized) type and adds it as fp32; the
   * LLM application always disables it (causal_lm.cpp:217-227), and so must a user of this layer */
  NNTR_THROW_IF(!disable_bias, exception::not_supported)
    << "TieWordEmbeddingHip as lm_head runs without bias: set disable_bias=true";
  (void)bias_dim;
}

void TieWordEmbeddingHip::forwarding(RunLayerContext &, bool) {}

void TieWordEmbeddingHip::incremental_forwarding(RunLayerContext &context, unsigned int from, unsigned int to,
                                                 bool training) {
  NNTR_THROW_IF(training, exception::not_supported) << "TieWordEmbeddingHip is an inference layer";
  NNTR_THROW_IF(to <= from, std::invalid_argument)
    << "incremental step [" << from << ", " << to << ") is empty";
  if (mode == Mode::embedding)
    step_embedding(context, from, to);
  else
    step_lmhead(context, from, to);
}

static float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ff, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400));
      bits = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ff) << 13;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | man << 13;
  } else {
    bits = sign | (exp + 127 - 15) << 23 | man << 13;
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

/* One row of a Q6_K table to fp32: per 256 values 128 low nibbles, 64 bytes of upper bit
 * pairs, 16 int8 scales and an fp16 super-scale; value = d * scale * (q - 32), the products
 * taken in that order (dequantize_row_q6_K, nntr_ggml_impl_quant.cpp:1291-1325). */
static void dequantize_q6_K_row(const uint8_t *blocks, float *y, unsigned int n) {
  for (unsigned int sb = 0; sb < n / 256; ++sb) {
    const uint8_t *ql = blocks + (size_t)sb * 210;
    const uint8_t *qh = ql + 128;
    const int8_t *sc = (const int8_t *)(qh + 64);
    uint16_t dbits;
    std::memcpy(&dbits, ql + 208, 2);
    const float d = half_bits_to_float(dbits);
    for (int half = 0; half < 2; ++half) {
      for (int l = 0; l < 32; ++l) {
        const int is = l / 16;
        const int q1 = (int)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
        const int q2 = (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
        const int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
        const int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
        y[l] = d * sc[is] * q1;
        y[l + 32] = d * sc[is + 2] * q2;
        y[l + 64] = d * sc[is + 4] * q3;
        y[l + 96] = d * sc[is + 6] * q4;
      }
      y += 128;
      ql += 64;
      qh += 32;
      sc += 8;
    }
  }
}

void TieWordEmbeddingHip::step_embedding(RunLayerContext &context, unsigned int from, unsigned int to) {
  Tensor &table = context.getWeight(weight_idx[Params::weight]);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  const Tdatatype wtype = table.getDataType();
  NNTR_THROW_IF(wtype != Tdatatype::Q6_K && wtype != Tdatatype::FP32, std::invalid_argument)
    << "Tieword embedding is not supported yet for the data type";
  const unsigned int iter = to - from;
  NNTR_THROW_IF(iter > input_.width() || iter > hidden_.height(), std::invalid_argument)
    << "incremental step of " << iter << " ids exceeds the input width " << input_.width();
  const size_t row_bytes = wtype == Tdatatype::Q6_K ? (size_t)210 * ((out_dim + 255) / 256) : (size_t)out_dim * 4;
  /* ids [0, to - from) of every batch entry, one output row each (tie_word_embedding.cpp:208-240) */
  for (unsigned int b = 0; b < input_.batch(); ++b) {
    const float *ids = input_.getData<float>() + (size_t)b * input_.getDim().getFeatureLen();
    float *out = hidden_.getData<float>() + (size_t)b * hidden_.getDim().getFeatureLen();
    for (unsigned int i = 0; i < iter; ++i) {
      const unsigned int id = static_cast<unsigned int>(ids[i]);
      if (id >= in_dim)
        throw std::invalid_argument("input word index is greater than in_dim");
      const uint8_t *row = table.getData<uint8_t>() + row_bytes * id;
      if (wtype == Tdatatype::Q6_K)
        dequantize_q6_K_row(row, out + (size_t)i * out_dim, out_dim);
      else
        std::memcpy(out + (size_t)i * out_dim, row, row_bytes);
    }
  }
}

void TieWordEmbeddingHip::step_lmhead(RunLayerContext &context, unsigned int from, unsigned int to) {
  Tensor &table = context.getWeight(weight_idx[Params::weight]);
  Tensor &input_ = context.getInput(SINGLE_INOUT_IDX);
  Tensor &hidden_ = context.getOutput(SINGLE_INOUT_IDX);
  const TensorDim input_dim = input_.getDim(), hidden_dim = hidden_.getDim();
  NNTR_THROW_IF(to > input_dim.height() && to - from != 1, std::invalid_argument)
    << "step end " << to << " exceeds the input height " << input_dim.height();
  const int dtype = hipq_dtype_of(table.getDataType());
  NNTR_THROW_IF(dtype < 0, std::invalid_argument)
    << "weight type is not supported for custom tie word embedding layer";
  /* N = the table's height, K = its width: dotQnK with trans_in (float_tensor.cpp:936-938) */
  const int64_t N = table.height(), K = table.width();
  NNTR_THROW_IF((int64_t)input_.width() != K || (int64_t)hidden_.width() != N, std::invalid_argument)
    << "lm_head: input width " << input_.width() << " and output width " << hidden_.width()
    << " do not match the table [" << N << " x " << K << "]";
  const hipq_host::WeightSpec spec{dtype, hipq_host::framework_layout(dtype), N, K};
  /* one row per batch entry: row 0 of a single-token step, else the step's last row
   * (tie_word_embedding.cpp:272-283) */
  const size_t row = to - from == 1 ? 0 : (size_t)(to - 1);
  for (unsigned int b = 0; b < input_dim.batch(); ++b) {
    const float *x = input_.getData<float>() + (size_t)b * input_dim.getFeatureLen() + row * input_.width();
    float *y = hidden_.getData<float>() + (size_t)b * hidden_dim.getFeatureLen() + row * hidden_.width();
    hipq_host::matmul(hipq_host::global_cache(), table.getData<uint8_t>(), spec, x, 1, K, y, N);
  }
}

void TieWordEmbeddingHip::calcDerivative(RunLayerContext &) {
  throw exception::not_supported("calcDerivative for Embedding layer is not supported");
}

void TieWordEmbeddingHip::calcGradient(RunLayerContext &) {}

void TieWordEmbeddingHip::read(std::ifstream &file, RunLayerContext &run_context, bool opt_var,
                               ml::train::ExecutionMode mode_, bool trainable,
                               TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                               bool read_from_offset, int file_fd) {
  Layer::read(file, run_context, opt_var, mode_, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset, file_fd);
  drop_device_copies(run_context);
}

void TieWordEmbeddingHip::read(ReadSource src, RunLayerContext &run_context, bool opt_var,
                               ml::train::ExecutionMode mode_, bool trainable,
                               TensorDim::DataType defineWeightDataType, bool fsu, size_t start_offset,
                               bool read_from_offset) {
  Layer::read(src, run_context, opt_var, mode_, trainable, defineWeightDataType, fsu, start_offset,
              read_from_offset);
  drop_device_copies(run_context);
}

} // namespace nntrainer
