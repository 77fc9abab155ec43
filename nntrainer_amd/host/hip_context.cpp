// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hip_context.cpp
 * @brief  HipContext implementation and the context plug-in record.
 */
#include "hip_context.h"

#include <algorithm>
#include <cctype>
#include <cstdio>
#include <sstream>

#include "fc_layer_hip.h"
#include "hip_mem_allocator.h"
#include "hipq_host.h"
#include "mlp_swiglu_layer_hip.h"
#include "moe_layer_hip.h"
#include "qkv_layer_hip.h"
#include "tie_word_embedding_hip.h"

namespace nntrainer {

static std::string to_lower(std::string s) {
  std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::tolower(c); });
  return s;
}

HipContext &HipContext::Global() {
  /* never destroyed, like every registered context (nntrainer/engine.h:52-57) */
  static HipContext *instance = new HipContext();
  instance->initialize();
  return *instance;
}

void HipContext::initialize() noexcept {
  try {
    std::call_once(init_flag, [this]() {
      device_ok = hipq_host::runtime_available();
      if (!device_ok)
        std::fprintf(stderr, "[HipContext] no usable HIP device (%s); layers will fail at forward time\n",
                     hipq_last_error());
      add_default_object();
      /* the pool that holds a model's tensors allocates through the context's allocator
       * (cl_context.cpp:83 sets the default one): page-locked memory here */
      getContextData()->setMemAllocator(std::make_shared<HipMemAllocator>());
    });
  } catch (const std::exception &e) {
    std::fprintf(stderr, "[HipContext] initialize failed: %s\n", e.what());
  } catch (...) {
    std::fprintf(stderr, "[HipContext] initialize failed\n");
  }
}

void HipContext::add_default_object() {
  registerFactory(nntrainer::createLayer<FullyConnectedLayerHip>, FullyConnectedLayerHip::type,
                  ml::train::LayerType::LAYER_FC);
  /* an application layer: it has no integer key in the framework either
   * (Applications/CausalLM/layers/qwen_moe_layer.h:107) */
  registerFactory(nntrainer::createLayer<MoELayerHip>, MoELayerHip::type, -1);
  /* the application's other layers on this path, under their own type keys
   * (qkv_layer.h:143, tie_word_embedding.h:140, qwen_moe_layer_cached.h:114-115,
   * gpt_oss_moe_layer.h:102, gpt_oss_moe_layer_cached.h:105-106) */
  registerFactory(nntrainer::createLayer<QKVLayerHip>, QKVLayerHip::type, -1);
  registerFactory(nntrainer::createLayer<TieWordEmbeddingHip>, TieWordEmbeddingHip::type, -1);
  registerFactory(nntrainer::createLayer<CachedSlimMoELayerHip>, CachedSlimMoELayerHip::type, -1);
  registerFactory(nntrainer::createLayer<GptOssMoELayerHip>, GptOssMoELayerHip::type, -1);
  registerFactory(nntrainer::createLayer<CachedSlimGptOssMoELayerHip>, CachedSlimGptOssMoELayerHip::type, -1);
  /* ffn_up + ffn_gate + swiglu of the application's MLP as one layer (no counterpart in the
   * framework: a graph opts in by creating it) */
  registerFactory(nntrainer::createLayer<MlpSwiGLULayerHip>, MlpSwiGLULayerHip::type, -1);
}

int HipContext::registerFactory(const FactoryType<Layer> factory, const std::string &key,
                                const int int_key) {
  if (!factory)
    throw std::invalid_argument("cannot register an empty factory");
  std::string assigned_key = key;
  if (assigned_key.empty()) {
    /* the type the factory's objects report, as the framework does */
    auto probe = factory({});
    assigned_key = probe->getType();
  }
  assigned_key = to_lower(assigned_key);

  const std::lock_guard<std::mutex> lock(factory_mutex);
  if (str_map.find(assigned_key) != str_map.end()) {
    std::stringstream ss;
    ss << "cannot register factory with already taken key: " << assigned_key;
    throw std::invalid_argument(ss.str());
  }
  if (int_key != -1 && int_map.find(int_key) != int_map.end()) {
    std::stringstream ss;
    ss << "cannot register factory with already taken int key: " << int_key;
    throw std::invalid_argument(ss.str());
  }
  int assigned_int_key = int_key;
  if (assigned_int_key == -1) {
    /* keys handed out here start above every built-in layer type */
    assigned_int_key = 1000;
    while (int_map.find(assigned_int_key) != int_map.end())
      ++assigned_int_key;
  }
  str_map[assigned_key] = factory;
  int_map[assigned_int_key] = assigned_key;
  return assigned_int_key;
}

Context::PtrType<Layer> HipContext::createLayerObject(const std::string &type,
                                                      const std::vector<std::string> &props) {
  FactoryType<Layer> factory;
  {
    const std::lock_guard<std::mutex> lock(factory_mutex);
    auto it = str_map.find(to_lower(type));
    if (it == str_map.end()) {
      std::stringstream ss;
      ss << "HipContext has no layer of type: " << type;
      throw exception::not_supported(ss.str());
    }
    factory = it->second;
  }
  return factory(props);
}

Context::PtrType<Layer> HipContext::createLayerObject(const int int_key,
                                                      const std::vector<std::string> &props) {
  std::string type;
  {
    const std::lock_guard<std::mutex> lock(factory_mutex);
    auto it = int_map.find(int_key);
    if (it == int_map.end()) {
      std::stringstream ss;
      ss << "HipContext has no layer with int key: " << int_key;
      throw exception::not_supported(ss.str());
    }
    type = it->second;
  }
  return createLayerObject(type, props);
}

} // namespace nntrainer

extern "C" {

static nntrainer::Context *create_hip_context() { return &nntrainer::HipContext::Global(); }

/* the context lives as long as the process; nothing to release per handle */
static void destroy_hip_context(nntrainer::Context *) {}

__attribute__((visibility("default"))) nntrainer::ContextPluggable ml_train_context_pluggable{
  create_hip_context, destroy_hip_context};
}
