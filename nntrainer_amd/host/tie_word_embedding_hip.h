// SPDX-License-Identifier: Apache-2.0
/**
 * @file   tie_word_embedding_hip.h
 * @brief  The layer that serves both ends of a model whose lm_head shares the embedding
 *         table: token look-up at the input, vocabulary projection at the output.
 *
 * Counterpart of causallm::TieWordEmbedding (Applications/CausalLM/layers/
 * tie_word_embedding.cpp; type key "tie_word_embeddings", tie_word_embedding.h:140). As there,
 * the mode follows from the properties (tie_word_embedding.cpp:43-51): with `unit` the layer is
 * the lm_head, without it the embedding (`in_dim`, `out_dim`).
 *  - lm_head (finalize_lmhead :102-164, incremental_forwarding_lmhead :252-303): the weight is
 *    requested transposed, [unit x in_width], so that it is the embedding table itself
 *    ("shared_from"); only the last row of a step is projected, hidden = input . W^T (+ bias).
 *    This is the product the GPU serves: for Qwen3 a Q6_K matrix of 151936 rows.
 *  - embedding (finalize_embedding :53-100, incremental_forwarding_embedding :183-250): row
 *    `token` of the table, dequantized for Q6_K or copied for FP32. A few rows of a table that
 *    lives in host memory: done on the host, as in the reference.
 */
#ifndef HIPQ_TIE_WORD_EMBEDDING_HIP_H
#define HIPQ_TIE_WORD_EMBEDDING_HIP_H

#include <array>
#include <string>
#include <vector>

#include "nntr_api.h"

namespace nntrainer {

class TieWordEmbeddingHip : public Layer {
public:
  TieWordEmbeddingHip() = default;
  ~TieWordEmbeddingHip() override = default;

  void finalize(InitLayerContext &context) override;
  /** a no-op, as in the reference (tie_word_embedding.cpp:171-172) */
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
  const std::string getType() const override { return TieWordEmbeddingHip::type; }
  bool supportBackwarding() const override { return false; }

  inline static const std::string type = "tie_word_embeddings";

private:
  enum Params { weight, bias };
  enum class Mode { embedding, lm_head };

  void finalize_embedding(InitLayerContext &context);
  void finalize_lmhead(InitLayerContext &context);
  void step_embedding(RunLayerContext &context, unsigned int from, unsigned int to);
  void step_lmhead(RunLayerContext &context, unsigned int from, unsigned int to);

  Mode mode = Mode::embedding;
  unsigned int in_dim = 0, out_dim = 0, unit = 0;
  bool disable_bias = false;
  std::array<unsigned int, 2> weight_idx = {0, 0};
};

} // namespace nntrainer

#endif /* HIPQ_TIE_WORD_EMBEDDING_HIP_H */
