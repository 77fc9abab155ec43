// SPDX-License-Identifier: Apache-2.0
/**
 * @file   layer_common.h
 * @brief  What the HIP layers share: the weight type codes and the hook that drops device
 *         copies of weights the framework has just rewritten.
 */
#ifndef HIPQ_LAYER_COMMON_H
#define HIPQ_LAYER_COMMON_H

#include "hipq_host.h"
#include "nntr_api.h"

namespace nntrainer {

/** code of include/hipq.h for a weight tensor type, -1 if the GPU path does not serve it */
inline int hipq_dtype_of(Tdatatype t) {
  switch (t) {
  case Tdatatype::Q4_0:
    return HIPQ_Q4_0;
  case Tdatatype::Q4_K:
    return HIPQ_Q4_K;
  case Tdatatype::Q6_K:
    return HIPQ_Q6_K;
  default:
    return -1;
  }
}

/** forget the device copies of all of a layer's weights (after Layer::read) */
inline void drop_device_copies(RunLayerContext &run_context) {
  for (unsigned int i = 0; i < run_context.getNumWeights(); ++i)
    hipq_host::global_cache().invalidate(run_context.getWeight(i).getData<uint8_t>());
}

} // namespace nntrainer

#endif /* HIPQ_LAYER_COMMON_H */
