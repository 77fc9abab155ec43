// SPDX-License-Identifier: Apache-2.0
/**
 * @file   host_selftest.cpp
 * @brief  Driver for the HIP context plug-in, built against the API stand-in.
 *
 * It loads the plug-in the way Engine::registerContext does
 * (nntrainer/engine.cpp:140-171): dlopen(RTLD_LAZY | RTLD_LOCAL), dlsym of
 * "ml_train_context_pluggable", createfunc(), getName(). Then, by mode:
 *   api                      checks that need no GPU: factory keys, error types,
 *                            properties, the tensors finalize() requests
 *   fc  <dtype> <K> <N> <batch> <height> <from> <to> <weight> <input> <bias|-> <out>
 *                            builds a fully_connected layer through the context,
 *                            fills its tensors from the files, runs forwarding
 *                            (from == to == 0) or incremental_forwarding and
 *                            writes the output tensor
 *   fcreload <dtype> <K> <N> <height> <weightA> <weightB> <input> <read|poke> <outA> <outB>
 *                            forwarding with weight A, then the weight tensor's bytes are replaced
 *                            by B in place -- through Layer::read as the model loader does it, or
 *                            behind the layer's back -- and forwarding runs again
 *   moe <dtype> <T> <H> <I> <E> <k> <incremental> <router> <experts> <input> <out>
 *                            the same for qwen_moe; <experts> holds up_e, gate_e,
 *                            down_e for e = 0.. in the order the layer requests them
 * The test suite compares the written outputs with expected values it computes itself.
 */
#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "nntr_api.h"

using namespace nntrainer;

static int failures = 0;
#define EXPECT(cond)                                                    \
  do {                                                                  \
    if (!(cond)) {                                                      \
      std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #cond);        \
      ++failures;                                                       \
    }                                                                   \
  } while (0)
#define EXPECT_THROW(stmt, Err)                                         \
  do {                                                                  \
    bool caught = false;                                                \
    try {                                                               \
      stmt;                                                             \
    } catch (const Err &) {                                             \
      caught = true;                                                    \
    } catch (...) {                                                     \
    }                                                                   \
    if (!caught) {                                                      \
      std::printf("FAIL %s:%d %s did not throw %s\n", __FILE__, __LINE__, #stmt, #Err); \
      ++failures;                                                       \
    }                                                                   \
  } while (0)

static Context *load_context(const std::string &lib_path) {
  void *handle = dlopen(lib_path.c_str(), RTLD_LAZY | RTLD_LOCAL);
  if (!handle) {
    std::printf("dlopen failed: %s\n", dlerror());
    std::exit(2);
  }
  auto *pluggable = reinterpret_cast<ContextPluggable *>(dlsym(handle, "ml_train_context_pluggable"));
  if (!pluggable) {
    std::printf("dlsym failed: %s\n", dlerror());
    std::exit(2);
  }
  Context *ctx = pluggable->createfunc();
  if (!ctx || ctx->getName().empty()) {
    std::printf("context has no name\n");
    std::exit(2);
  }
  return ctx;
}

static Tdatatype dtype_of(const std::string &s) {
  if (s == "q4_0")
    return Tdatatype::Q4_0;
  if (s == "q4_K")
    return Tdatatype::Q4_K;
  if (s == "q6_K")
    return Tdatatype::Q6_K;
  std::printf("unknown dtype %s\n", s.c_str());
  std::exit(2);
}

static void read_into(const std::string &path, void *dst, size_t bytes) {
  std::ifstream f(path, std::ios::binary);
  f.read(reinterpret_cast<char *>(dst), bytes);
  if ((size_t)f.gcount() != bytes) {
    std::printf("%s: expected %zu bytes, got %zu\n", path.c_str(), bytes, (size_t)f.gcount());
    std::exit(2);
  }
}

static void write_from(const std::string &path, const void *src, size_t bytes) {
  std::ofstream f(path, std::ios::binary);
  f.write(reinterpret_cast<const char *>(src), bytes);
}

static int run_api(Context *ctx) {
  EXPECT(ctx->getName() == "gpu");
  EXPECT(ctx->getContextData() != nullptr);

  /* factory keys: string (case-insensitive) and integer */
  auto fc = ctx->createLayerObject("fully_connected", {"unit=512", "disable_bias=true"});
  EXPECT(fc && fc->getType() == "fully_connected");
  auto fc2 = ctx->createLayerObject("Fully_Connected", {"unit=8"});
  EXPECT(fc2 && fc2->getType() == "fully_connected");
  auto fc3 = ctx->createLayerObject(ml::train::LayerType::LAYER_FC, {"unit=8"});
  EXPECT(fc3 && fc3->getType() == "fully_connected");
  auto moe = ctx->createLayerObject(
    "qwen_moe", {"num_experts=4", "num_experts_per_token=2", "unit=256", "moe_activation=swish"});
  EXPECT(moe && moe->getType() == "qwen_moe");
  EXPECT_THROW(ctx->createLayerObject("conv2d", {}), exception::not_supported);
  EXPECT_THROW(ctx->createLayerObject(424242, {}), exception::not_supported);

  /* properties */
  EXPECT_THROW(ctx->createLayerObject("fully_connected", {"unit=0"}), std::invalid_argument);
  EXPECT_THROW(ctx->createLayerObject("fully_connected", {"unit=abc"}), std::invalid_argument);
  EXPECT_THROW(ctx->createLayerObject("fully_connected", {"no_such_prop=1"}), std::invalid_argument);
  EXPECT_THROW(ctx->createLayerObject("fully_connected", {"unit"}), std::invalid_argument);
  EXPECT_THROW(ctx->createLayerObject("fully_connected", {"unit=8", "lora_rank=4"}),
               exception::not_supported);
  EXPECT_THROW(ctx->createLayerObject("qwen_moe", {"moe_activation=relu"}), exception::not_supported);
  EXPECT(!fc->supportBackwarding() && !moe->supportBackwarding());

  /* finalize of fully_connected: output dims and requested tensors */
  {
    InitLayerContext ic({TensorDim(1, 1, 7, 1024)}, "fc0", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    fc->finalize(ic);
    EXPECT(ic.getOutputDimensions().size() == 1);
    EXPECT(ic.getOutputDimensions()[0] == TensorDim(1, 1, 7, 512));
    EXPECT(ic.getWeightRequests().size() == 1); /* bias disabled */
    EXPECT(ic.getWeightRequests()[0].dim == TensorDim(1, 1, 1024, 512));
    EXPECT(ic.getWeightRequests()[0].dim.getDataType() == Tdatatype::Q4_K);
    EXPECT(ic.getWeightRequests()[0].name == "fc0:weight");
  }
  {
    InitLayerContext ic({TensorDim(2, 1, 3, 256)}, "fc1", Tformat::NCHW, Tdatatype::Q6_K, Tdatatype::FP32);
    fc2->finalize(ic);
    EXPECT(ic.getWeightRequests().size() == 2);
    EXPECT(ic.getWeightRequests()[1].dim == TensorDim(1, 1, 1, 8));
    EXPECT(ic.getWeightRequests()[1].dim.getDataType() == Tdatatype::FP32);
  }
  {
    /* two inputs, unsupported weight type, width not a multiple of the block */
    InitLayerContext two({TensorDim(1, 1, 1, 256), TensorDim(1, 1, 1, 256)}, "x", Tformat::NCHW,
                         Tdatatype::Q4_K, Tdatatype::FP32);
    EXPECT_THROW(fc3->finalize(two), std::invalid_argument);
    InitLayerContext f32({TensorDim(1, 1, 1, 256)}, "x", Tformat::NCHW, Tdatatype::FP32, Tdatatype::FP32);
    EXPECT_THROW(fc3->finalize(f32), exception::not_supported);
    InitLayerContext odd({TensorDim(1, 1, 1, 200)}, "x", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    EXPECT_THROW(fc3->finalize(odd), std::invalid_argument);
    EXPECT_THROW(ctx->createLayerObject("fully_connected", {})->finalize(f32), std::invalid_argument);
  }
  /* finalize of qwen_moe: router first, then up, gate, down per expert */
  {
    InitLayerContext ic({TensorDim(1, 1, 5, 512)}, "moe0", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    moe->finalize(ic);
    const auto &w = ic.getWeightRequests();
    EXPECT(w.size() == 1 + 3 * 4);
    EXPECT(w[0].name == "moe0:gate" && w[0].dim == TensorDim(1, 1, 512, 4) &&
           w[0].dim.getDataType() == Tdatatype::FP32);
    EXPECT(w[1].name == "moe0:expert_up_0" && w[1].dim == TensorDim(1, 1, 512, 256));
    EXPECT(w[2].name == "moe0:expert_gate_0" && w[2].dim == TensorDim(1, 1, 512, 256));
    EXPECT(w[3].name == "moe0:expert_down_0" && w[3].dim == TensorDim(1, 1, 256, 512));
    EXPECT(w[12].name == "moe0:expert_down_3");
    EXPECT(ic.getTensorRequests().size() == 2);
    EXPECT(ic.getTensorRequests()[0].dim == TensorDim(5, 1, 1, 4));
    EXPECT(ic.getTensorRequests()[1].dim == TensorDim(4, 1, 2, 5));
    EXPECT(ic.getOutputDimensions()[0] == TensorDim(1, 1, 5, 512));
  }
  {
    auto m = ctx->createLayerObject("qwen_moe", {"num_experts=4", "num_experts_per_token=2", "unit=256"});
    InitLayerContext ic({TensorDim(1, 1, 5, 512)}, "m", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    EXPECT_THROW(m->finalize(ic), std::runtime_error); /* activation not set */
    auto k = ctx->createLayerObject(
      "qwen_moe", {"num_experts=2", "num_experts_per_token=3", "unit=256", "moe_activation=swish"});
    EXPECT_THROW(k->finalize(ic), std::invalid_argument);
  }
  /* inference only */
  {
    RunLayerContext rc;
    EXPECT_THROW(fc->calcDerivative(rc), exception::not_supported);
    EXPECT_THROW(moe->calcDerivative(rc), exception::not_supported);
  }
  std::printf(failures ? "API CHECKS FAILED (%d)\n" : "API CHECKS PASSED\n", failures);
  return failures ? 1 : 0;
}

static int run_fc(Context *ctx, char **a) {
  const std::string dt = a[0];
  const unsigned K = std::atoi(a[1]), N = std::atoi(a[2]), batch = std::atoi(a[3]),
                 height = std::atoi(a[4]), from = std::atoi(a[5]), to = std::atoi(a[6]);
  const std::string wpath = a[7], ipath = a[8], bpath = a[9], opath = a[10];
  const bool has_bias = bpath != "-";
  std::vector<std::string> props = {"unit=" + std::to_string(N)};
  props.push_back(has_bias ? "disable_bias=false" : "disable_bias=true");
  auto layer = ctx->createLayerObject("fully_connected", props);
  InitLayerContext ic({TensorDim(batch, 1, height, K)}, "fc", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  read_into(wpath, rc.getWeight(0).getData<uint8_t>(), mirror_tensor_bytes(rc.getWeight(0).getDim()));
  if (has_bias)
    read_into(bpath, rc.getWeight(1).getData<float>(), (size_t)N * 4);
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)batch * height * K * 4);
  /* rows a step does not write keep this value */
  float *out = rc.getOutput(0).getData<float>();
  for (size_t i = 0; i < (size_t)batch * height * N; ++i)
    out[i] = -12345.f;
  if (from == 0 && to == 0)
    layer->forwarding(rc, false);
  else
    layer->incremental_forwarding(rc, from, to, false);
  write_from(opath, out, (size_t)batch * height * N * 4);
  std::printf("FC DONE\n");
  return 0;
}

static int run_fc_reload(Context *ctx, char **a) {
  const std::string dt = a[0];
  const unsigned K = std::atoi(a[1]), N = std::atoi(a[2]), height = std::atoi(a[3]);
  const std::string wa = a[4], wb = a[5], ipath = a[6], how = a[7], oa = a[8], ob = a[9];
  auto layer = ctx->createLayerObject("fully_connected", {"unit=" + std::to_string(N), "disable_bias=true"});
  InitLayerContext ic({TensorDim(1, 1, height, K)}, "fc", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  const size_t wbytes = mirror_tensor_bytes(rc.getWeight(0).getDim());
  read_into(wa, rc.getWeight(0).getData<uint8_t>(), wbytes);
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)height * K * 4);
  float *out = rc.getOutput(0).getData<float>();
  layer->forwarding(rc, false);
  write_from(oa, out, (size_t)height * N * 4);
  if (how == "read") {
    std::ifstream f(wb, std::ios::binary);
    layer->read(f, rc, false, ml::train::ExecutionMode::INFERENCE, false, dtype_of(dt), false);
  } else {
    read_into(wb, rc.getWeight(0).getData<uint8_t>(), wbytes);
  }
  layer->forwarding(rc, false);
  write_from(ob, out, (size_t)height * N * 4);
  std::printf("FC RELOAD DONE\n");
  return 0;
}

static int run_moe(Context *ctx, char **a) {
  const std::string dt = a[0];
  const unsigned T = std::atoi(a[1]), H = std::atoi(a[2]), I = std::atoi(a[3]), E = std::atoi(a[4]),
                 k = std::atoi(a[5]), incremental = std::atoi(a[6]);
  const std::string rpath = a[7], epath = a[8], ipath = a[9], opath = a[10];
  auto layer = ctx->createLayerObject("qwen_moe", {"num_experts=" + std::to_string(E),
                                                    "num_experts_per_token=" + std::to_string(k),
                                                    "unit=" + std::to_string(I), "moe_activation=swish"});
  InitLayerContext ic({TensorDim(1, 1, T, H)}, "moe", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  read_into(rpath, rc.getWeight(0).getData<float>(), (size_t)H * E * 4);
  {
    std::ifstream f(epath, std::ios::binary);
    for (unsigned i = 1; i < rc.getNumWeights(); ++i) {
      const size_t bytes = mirror_tensor_bytes(rc.getWeight(i).getDim());
      f.read(rc.getWeight(i).getData<char>(), bytes);
      if ((size_t)f.gcount() != bytes) {
        std::printf("%s: short read at weight %u\n", epath.c_str(), i);
        return 2;
      }
    }
  }
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)T * H * 4);
  if (incremental)
    layer->incremental_forwarding(rc, 0, T, false);
  else
    layer->forwarding(rc, false);
  write_from(opath, rc.getOutput(0).getData<float>(), (size_t)T * H * 4);
  std::printf("MOE DONE\n");
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 3) {
    std::printf("usage: %s <plugin.so> api | fc ... | moe ...\n", argv[0]);
    return 2;
  }
  try {
    Context *ctx = load_context(argv[1]);
    const std::string mode = argv[2];
    if (mode == "api")
      return run_api(ctx);
    if (mode == "fc" && argc == 14)
      return run_fc(ctx, argv + 3);
    if (mode == "moe" && argc == 14)
      return run_moe(ctx, argv + 3);
    if (mode == "fcreload" && argc == 13)
      return run_fc_reload(ctx, argv + 3);
    std::printf("bad arguments for mode %s (argc %d)\n", mode.c_str(), argc);
    return 2;
  } catch (const std::exception &e) {
    std::printf("EXCEPTION %s\n", e.what());
    return 3;
  }
}
