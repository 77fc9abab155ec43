// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hip_context.h
 * @brief  HipContext: the compute-engine context that serves layers created
 *         with engine=gpu from HIP kernels on an AMD GPU.
 *
 * It takes the place ClContext has in the framework (nntrainer/cl_context.h:47-246,
 * nntrainer/cl_context.cpp:60-171): a process-wide object behind Global(), a
 * factory map for layers keyed by lower-cased type string and by integer key,
 * getName() == "gpu" so that Engine::parseComputeEngine (nntrainer/engine.cpp:66-84)
 * routes `engine=gpu` layers here, and the plug-in record
 * `ml_train_context_pluggable` that Engine::registerContext dlsym()s
 * (nntrainer/engine.cpp:140-171, nntrainer/context.h:225-240).
 */
#ifndef HIPQ_HIP_CONTEXT_H
#define HIPQ_HIP_CONTEXT_H

#include <mutex>
#include <string>

#include "nntr_api.h"

namespace nntrainer {

class HipContext : public Context {
public:
  HipContext() : Context(std::make_shared<ContextData>()) {}
  ~HipContext() override = default;

  /** the one context of the process; registers the default layers on first use */
  static HipContext &Global();

  /** brings the device up and registers the layers; logs and returns instead of
   *  throwing when no GPU is usable (cl_context.cpp:70-90) */
  void initialize() noexcept;

  int init() override {
    initialize();
    return 0;
  }

  std::string getName() override { return "gpu"; }

  /** true once a HIP device is usable; layers can still be created without */
  bool deviceAvailable() const { return device_ok; }

  /**
   * @brief register a layer factory under a string key and an integer key
   * @throws std::invalid_argument if the key (case-insensitive) or the integer
   *         key is already taken (cl_context.cpp:132-171)
   * @return the integer key in use (assigned when int_key == -1)
   */
  int registerFactory(const FactoryType<Layer> factory, const std::string &key = "",
                      const int int_key = -1);
  int registerFactory(const PtrFactoryType<Layer> factory, const std::string &key = "",
                      const int int_key = -1) {
    FactoryType<Layer> f = factory;
    return registerFactory(f, key, int_key);
  }

  /** @throws exception::not_supported for an unknown type (cl_context.h:139-175) */
  PtrType<Layer> createLayerObject(const std::string &type,
                                   const std::vector<std::string> &props = {}) override;
  PtrType<Layer> createLayerObject(const int int_key,
                                   const std::vector<std::string> &props = {}) override;

private:
  void add_default_object();

  std::mutex factory_mutex;
  std::once_flag init_flag;
  bool device_ok = false;
  StrIndexType<Layer> str_map;
  IntIndexType int_map;
};

} // namespace nntrainer

#endif /* HIPQ_HIP_CONTEXT_H */
