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
 *   moe <dtype> <T> <H> <I> <E> <k> <incremental> <router> <experts> <input> <out> [<experts_b> <out_b>]
 *                            the same for qwen_moe; <experts> holds up_e, gate_e,
 *                            down_e for e = 0.. in the order the layer requests them; with <experts_b> the
 *                            expert tensors are then overwritten in place with that file and the layer runs again
 *   moex <type> <dtype> <T> <H> <I> <E> <k> <incremental> <weights> <input> <out>
 *                            any of the MoE layer types; <weights> holds every weight in the order
 *                            the layer requests them and is loaded through Layer::read (which is how
 *                            virtual tensors get their bytes)
 *   qkv <dtype> <K> <Nq> <Nk> <Nv> <height> <from> <to> <weights> <input> <out>
 *                            qkv_layer; <weights> holds q, k, v; <out> the three outputs one after
 *                            the other
 *   mlp <dtype> <K> <unit> <batch> <height> <from> <to> <weights> <input> <out> [<down_unit>]
 *                            mlp_swiglu; <weights> holds the up then the gate matrix, with <down_unit> the down
 *                            projection's after them (the whole MLP as one layer)
 *   lmhead <dtype> <K> <unit> <batch> <height> <from> <to> <table> <input> <out>
 *   embed <dtype> <in_dim> <out_dim> <batch> <width> <from> <to> <table> <ids> <out>
 *                            tie_word_embeddings in its two modes
 *   c5layer <iterations>     times the quantized FCs of one Qwen3-0.6B-shaped decoder layer (hidden 1024,
 *                            Q 2048, K and V 1024, feed-forward 3072, Q4_0) through the layer API, every call
 *                            synchronous on host tensors as the framework makes it: as seven fully_connected
 *                            layers (what an unchanged graph gives) and as qkv_layer + fully_connected +
 *                            mlp_swiglu + fully_connected; one decode row and a prefill of 512 rows; tensors in
 *                            ordinary memory and in memory of the context's allocator. Prints one JSON object.
 *                            Weights are pseudo-random blocks: the mode measures time, the other modes results.
 *   moelayer <iterations>    the same for one qwen_moe layer of the Qwen3-30B-A3B shape (hidden 2048, 128 experts of
 *                            768, top 8, Q4_K): one decode token and a chunk of 64 tokens per call
 * The test suite compares the written outputs with expected values it computes itself.
 */
#include <dlfcn.h>

#include <chrono>
#include <cstring>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <memory>
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
  if (s == "fp32")
    return Tdatatype::FP32;
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
  /* the context publishes an allocator (cl_context.cpp:83); it works without a device too */
  {
    auto ma = ctx->getContextData()->getMemAllocator();
    EXPECT(ma != nullptr);
    if (ma) {
      EXPECT(ma->getName() == "gpu");
      void *p = nullptr;
      ma->alloc(&p, 4096, 64);
      EXPECT(p != nullptr);
      bool zero = p != nullptr;
      for (int i = 0; zero && i < 4096; ++i)
        zero = static_cast<unsigned char *>(p)[i] == 0;
      EXPECT(zero);
      ma->free(p);
      ma->free(nullptr);
    }
  }

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
  /* qkv_layer: three weights in q, k, v order, three outputs (qkv_layer.cpp:43-110) */
  {
    auto qkv = ctx->createLayerObject("qkv_layer", {"q_unit=512", "k_unit=256", "v_unit=128"});
    EXPECT(qkv && qkv->getType() == "qkv_layer");
    InitLayerContext ic({TensorDim(1, 1, 9, 1024)}, "l0_qkv", Tformat::NCHW, Tdatatype::Q4_0, Tdatatype::FP32);
    qkv->finalize(ic);
    const auto &w = ic.getWeightRequests();
    EXPECT(w.size() == 3);
    EXPECT(w[0].name == "l0_qkv:qweight" && w[0].dim == TensorDim(1, 1, 1024, 512));
    EXPECT(w[1].name == "l0_qkv:kweight" && w[1].dim == TensorDim(1, 1, 1024, 256));
    EXPECT(w[2].name == "l0_qkv:vweight" && w[2].dim == TensorDim(1, 1, 1024, 128));
    EXPECT(w[2].dim.getDataType() == Tdatatype::Q4_0);
    EXPECT(ic.getOutputDimensions().size() == 3);
    EXPECT(ic.getOutputDimensions()[0] == TensorDim(1, 1, 9, 512));
    EXPECT(ic.getOutputDimensions()[2] == TensorDim(1, 1, 9, 128));
    EXPECT_THROW(ctx->createLayerObject("qkv_layer", {"q_unit=8", "k_unit=8"})->finalize(ic), std::invalid_argument);
    EXPECT_THROW(ctx->createLayerObject("qkv_layer", {"unit=8"}), std::invalid_argument);
  }
  /* tie_word_embeddings: the mode follows from the properties (tie_word_embedding.cpp:43-51) */
  {
    auto head = ctx->createLayerObject("tie_word_embeddings", {"unit=4096", "disable_bias=true"});
    EXPECT(head && head->getType() == "tie_word_embeddings");
    InitLayerContext ic({TensorDim(1, 1, 5, 1024)}, "out", Tformat::NCHW, Tdatatype::Q6_K, Tdatatype::FP32);
    head->finalize(ic);
    EXPECT(ic.getWeightRequests().size() == 1);
    EXPECT(ic.getWeightRequests()[0].name == "out:Embedding");
    EXPECT(ic.getWeightRequests()[0].dim == TensorDim(1, 1, 4096, 1024)); /* the table: unit rows */
    EXPECT(ic.getOutputDimensions()[0] == TensorDim(1, 1, 5, 4096));
    auto emb = ctx->createLayerObject("tie_word_embeddings", {"in_dim=4096", "out_dim=1024"});
    InitLayerContext ie({TensorDim(1, 1, 1, 7)}, "emb", Tformat::NCHW, Tdatatype::Q6_K, Tdatatype::FP32);
    emb->finalize(ie);
    EXPECT(ie.getWeightRequests()[0].dim == TensorDim(1, 1, 4096, 1024));
    EXPECT(ie.getOutputDimensions()[0] == TensorDim(1, 1, 7, 1024));
    auto biased = ctx->createLayerObject("tie_word_embeddings", {"unit=4096"});
    EXPECT_THROW(biased->finalize(ic), exception::not_supported);
  }
  /* the other MoE layers: request order and virtual tensors */
  {
    auto cached = ctx->createLayerObject(
      "moe_cached_slim", {"num_experts=4", "num_experts_per_token=2", "unit=256", "moe_activation=swish"});
    EXPECT(cached && cached->getType() == "moe_cached_slim");
    InitLayerContext ic({TensorDim(1, 1, 5, 512)}, "m", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    cached->finalize(ic);
    EXPECT(ic.getWeightRequests().size() == 13);
    EXPECT(!ic.getWeightRequests()[0].is_virtual && ic.getWeightRequests()[1].is_virtual &&
           ic.getWeightRequests()[12].is_virtual);
    auto oss = ctx->createLayerObject("gpt_oss_moe", {"num_experts=4", "num_experts_per_token=2", "unit=256"});
    EXPECT(oss && oss->getType() == "gpt_oss_moe");
    InitLayerContext io({TensorDim(1, 1, 5, 512)}, "g", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    oss->finalize(io);
    const auto &w = io.getWeightRequests();
    EXPECT(w.size() == 2 + 6 * 4);
    EXPECT(w[0].name == "g:gate" && w[1].name == "g:gate_bias" && w[1].dim == TensorDim(1, 1, 1, 4));
    EXPECT(w[2].name == "g:expert_up_0" && w[3].name == "g:expert_up_bias_0" && w[3].dim == TensorDim(1, 1, 1, 256));
    EXPECT(w[4].name == "g:expert_gate_0" && w[5].name == "g:expert_gate_bias_0");
    EXPECT(w[6].name == "g:expert_down_0" && w[7].name == "g:expert_down_bias_0" &&
           w[7].dim == TensorDim(1, 1, 1, 512) && w[7].dim.getDataType() == Tdatatype::FP32);
    EXPECT(!w[2].is_virtual);
    auto both = ctx->createLayerObject("gpt_oss_moe_slim_cached",
                                       {"num_experts=4", "num_experts_per_token=2", "unit=256"});
    InitLayerContext ib({TensorDim(1, 1, 5, 512)}, "b", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    both->finalize(ib);
    EXPECT(ib.getWeightRequests().size() == 26 && ib.getWeightRequests()[3].is_virtual &&
           !ib.getWeightRequests()[1].is_virtual);
  }
  /* mlp_swiglu: up then gate, the order of the two FCs' weights in a model file */
  {
    auto mlp = ctx->createLayerObject("mlp_swiglu", {"unit=3072", "disable_bias=true"});
    EXPECT(mlp && mlp->getType() == "mlp_swiglu");
    InitLayerContext ic({TensorDim(1, 1, 4, 1024)}, "l0_ffn", Tformat::NCHW, Tdatatype::Q4_0, Tdatatype::FP32);
    mlp->finalize(ic);
    EXPECT(ic.getWeightRequests().size() == 2);
    EXPECT(ic.getWeightRequests()[0].name == "l0_ffn:up_weight" && ic.getWeightRequests()[1].name == "l0_ffn:gate_weight");
    EXPECT(ic.getWeightRequests()[1].dim == TensorDim(1, 1, 1024, 3072));
    EXPECT(ic.getOutputDimensions()[0] == TensorDim(1, 1, 4, 3072));
    EXPECT_THROW(ctx->createLayerObject("mlp_swiglu", {"unit=8", "disable_bias=false"}), exception::not_supported);
    /* with down_unit: the whole MLP, the down projection's weight third, the output as wide as the model */
    auto whole = ctx->createLayerObject("mlp_swiglu", {"unit=3072", "down_unit=1024", "disable_bias=true"});
    InitLayerContext iw({TensorDim(1, 1, 4, 1024)}, "l0_ffn", Tformat::NCHW, Tdatatype::Q4_0, Tdatatype::FP32);
    whole->finalize(iw);
    EXPECT(iw.getWeightRequests().size() == 3 && iw.getWeightRequests()[2].name == "l0_ffn:down_weight");
    EXPECT(iw.getWeightRequests()[2].dim == TensorDim(1, 1, 3072, 1024));
    EXPECT(iw.getOutputDimensions()[0] == TensorDim(1, 1, 4, 1024));
    auto odd = ctx->createLayerObject("mlp_swiglu", {"unit=3000", "down_unit=1024"});
    InitLayerContext io({TensorDim(1, 1, 4, 1024)}, "odd", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
    EXPECT_THROW(odd->finalize(io), std::invalid_argument);
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

static int run_moe(Context *ctx, char **a, char **second) {
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
  if (second) { /* other experts at the same addresses: the layer must not serve the old device copies */
    std::ifstream f(second[0], std::ios::binary);
    for (unsigned i = 1; i < rc.getNumWeights(); ++i)
      f.read(rc.getWeight(i).getData<char>(), mirror_tensor_bytes(rc.getWeight(i).getDim()));
    if (incremental)
      layer->incremental_forwarding(rc, 0, T, false);
    else
      layer->forwarding(rc, false);
    write_from(second[1], rc.getOutput(0).getData<float>(), (size_t)T * H * 4);
  }
  std::printf("MOE DONE\n");
  return 0;
}

static int run_moex(Context *ctx, char **a) {
  const std::string type = a[0], dt = a[1];
  const unsigned T = std::atoi(a[2]), H = std::atoi(a[3]), I = std::atoi(a[4]), E = std::atoi(a[5]),
                 k = std::atoi(a[6]), incremental = std::atoi(a[7]);
  const std::string wpath = a[8], ipath = a[9], opath = a[10];
  std::vector<std::string> props = {"num_experts=" + std::to_string(E), "num_experts_per_token=" + std::to_string(k),
                                    "unit=" + std::to_string(I)};
  if (type.find("gpt_oss") == std::string::npos)
    props.push_back("moe_activation=swish");
  auto layer = ctx->createLayerObject(type, props);
  InitLayerContext ic({TensorDim(1, 1, T, H)}, "moe", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  {
    std::ifstream f(wpath, std::ios::binary);
    layer->read(f, rc, false, ml::train::ExecutionMode::INFERENCE, false, dtype_of(dt), false);
  }
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)T * H * 4);
  float *out = rc.getOutput(0).getData<float>();
  for (size_t i = 0; i < (size_t)T * H; ++i)
    out[i] = -12345.f;
  for (int rep = 0; rep < 2; ++rep) { /* the second run finds cached experts resident */
    if (incremental)
      layer->incremental_forwarding(rc, 0, T, false);
    else
      layer->forwarding(rc, false);
  }
  write_from(opath, out, (size_t)T * H * 4);
  /* a cached layer leaves its virtual expert tensors deactivated */
  unsigned active_virtual = 0;
  for (unsigned i = 0; i < rc.getNumWeights(); ++i)
    if (ic.getWeightRequests()[i].is_virtual && rc.getWeight(i).getData<uint8_t>() != nullptr)
      ++active_virtual;
  std::printf("MOEX DONE active_virtual=%u\n", active_virtual);
  return 0;
}

static int run_qkv(Context *ctx, char **a) {
  const std::string dt = a[0];
  const unsigned K = std::atoi(a[1]), Nq = std::atoi(a[2]), Nk = std::atoi(a[3]), Nv = std::atoi(a[4]),
                 height = std::atoi(a[5]), from = std::atoi(a[6]), to = std::atoi(a[7]);
  const std::string wpath = a[8], ipath = a[9], opath = a[10];
  auto layer = ctx->createLayerObject("qkv_layer", {"q_unit=" + std::to_string(Nq), "k_unit=" + std::to_string(Nk),
                                                     "v_unit=" + std::to_string(Nv)});
  InitLayerContext ic({TensorDim(1, 1, height, K)}, "qkv", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  {
    std::ifstream f(wpath, std::ios::binary);
    layer->read(f, rc, false, ml::train::ExecutionMode::INFERENCE, false, dtype_of(dt), false);
  }
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)height * K * 4);
  const unsigned N[3] = {Nq, Nk, Nv};
  for (int o = 0; o < 3; ++o) {
    float *out = rc.getOutput(o).getData<float>();
    for (size_t i = 0; i < (size_t)height * N[o]; ++i)
      out[i] = -12345.f; /* rows a step does not write keep this value */
  }
  layer->forwarding(rc, false); /* a no-op in this layer */
  layer->incremental_forwarding(rc, from, to, false);
  std::ofstream f(opath, std::ios::binary);
  for (int o = 0; o < 3; ++o)
    f.write(rc.getOutput(o).getData<char>(), (size_t)height * N[o] * 4);
  std::printf("QKV DONE\n");
  return 0;
}

static int run_mlp(Context *ctx, char **a, unsigned down_unit) {
  const std::string dt = a[0];
  const unsigned K = std::atoi(a[1]), N = std::atoi(a[2]), batch = std::atoi(a[3]), height = std::atoi(a[4]),
                 from = std::atoi(a[5]), to = std::atoi(a[6]);
  const std::string wpath = a[7], ipath = a[8], opath = a[9];
  std::vector<std::string> props = {"unit=" + std::to_string(N), "disable_bias=true"};
  if (down_unit)
    props.push_back("down_unit=" + std::to_string(down_unit));
  const unsigned W = down_unit ? down_unit : N; /* the output's width */
  auto layer = ctx->createLayerObject("mlp_swiglu", props);
  InitLayerContext ic({TensorDim(batch, 1, height, K)}, "mlp", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  {
    std::ifstream f(wpath, std::ios::binary);
    layer->read(f, rc, false, ml::train::ExecutionMode::INFERENCE, false, dtype_of(dt), false);
  }
  read_into(ipath, rc.getInput(0).getData<float>(), (size_t)batch * height * K * 4);
  float *out = rc.getOutput(0).getData<float>();
  for (size_t i = 0; i < (size_t)batch * height * W; ++i)
    out[i] = -12345.f;
  if (from == 0 && to == 0)
    layer->forwarding(rc, false);
  else
    layer->incremental_forwarding(rc, from, to, false);
  write_from(opath, out, (size_t)batch * height * W * 4);
  std::printf("MLP DONE\n");
  return 0;
}

static int run_tie(Context *ctx, bool lmhead, char **a) {
  const std::string dt = a[0];
  const unsigned d0 = std::atoi(a[1]), d1 = std::atoi(a[2]), batch = std::atoi(a[3]), len = std::atoi(a[4]),
                 from = std::atoi(a[5]), to = std::atoi(a[6]);
  const std::string tpath = a[7], ipath = a[8], opath = a[9];
  std::unique_ptr<Layer> layer;
  std::vector<TensorDim> in;
  if (lmhead) { /* d0 = K, d1 = unit, len = height */
    layer = ctx->createLayerObject("tie_word_embeddings", {"unit=" + std::to_string(d1), "disable_bias=true"});
    in = {TensorDim(batch, 1, len, d0)};
  } else { /* d0 = in_dim, d1 = out_dim, len = ids per batch entry */
    layer = ctx->createLayerObject("tie_word_embeddings",
                                   {"in_dim=" + std::to_string(d0), "out_dim=" + std::to_string(d1)});
    in = {TensorDim(batch, 1, 1, len)};
  }
  InitLayerContext ic(in, "tie", Tformat::NCHW, dtype_of(dt), Tdatatype::FP32);
  layer->finalize(ic);
  RunLayerContext rc(ic);
  read_into(tpath, rc.getWeight(0).getData<uint8_t>(), mirror_tensor_bytes(rc.getWeight(0).getDim()));
  read_into(ipath, rc.getInput(0).getData<float>(), rc.getInput(0).size() * 4);
  float *out = rc.getOutput(0).getData<float>();
  const size_t n_out = rc.getOutput(0).size();
  for (size_t i = 0; i < n_out; ++i)
    out[i] = -12345.f;
  layer->incremental_forwarding(rc, from, to, false);
  write_from(opath, out, n_out * 4);
  std::printf("TIE DONE\n");
  return 0;
}

/* ---- c5layer ------------------------------------------------------------------------- */
namespace {
struct BuiltLayer {
  std::unique_ptr<Layer> layer;
  std::unique_ptr<InitLayerContext> ic;
  std::unique_ptr<RunLayerContext> rc;
  unsigned n_out = 1;
};

/* x8-repacked Q4_0 as the layer's weight tensor holds it: groups of 144 bytes, eight fp16 scales
 * (2^-8 here), then 128 bytes of nibbles */
void fill_q4_0x8(uint8_t *p, size_t bytes, uint32_t seed) {
  uint32_t x = seed * 2654435761u + 12345u;
  for (size_t g = 0; g + 144 <= bytes; g += 144) {
    for (int i = 0; i < 8; ++i) {
      p[g + 2 * i] = 0x00;
      p[g + 2 * i + 1] = 0x1c;
    }
    for (int i = 16; i < 144; ++i) {
      x = x * 1664525u + 1013904223u;
      p[g + i] = (uint8_t)(x >> 24);
    }
  }
}

BuiltLayer build(Context *ctx, const std::string &type, const std::vector<std::string> &props, unsigned height,
                 unsigned K, unsigned n_out, uint32_t seed, const std::shared_ptr<MemAllocator> &ma) {
  BuiltLayer b;
  b.layer = ctx->createLayerObject(type, props);
  b.ic = std::make_unique<InitLayerContext>(std::vector<TensorDim>{TensorDim(1, 1, height, K)}, type, Tformat::NCHW,
                                            Tdatatype::Q4_0, Tdatatype::FP32);
  b.layer->finalize(*b.ic);
  b.rc = std::make_unique<RunLayerContext>(*b.ic);
  b.n_out = n_out;
  for (unsigned i = 0; i < b.rc->getNumWeights(); ++i)
    fill_q4_0x8(b.rc->getWeight(i).getData<uint8_t>(), mirror_tensor_bytes(b.rc->getWeight(i).getDim()), seed + i);
  float *in = b.rc->getInput(0).getData<float>();
  for (size_t i = 0; i < (size_t)height * K; ++i)
    in[i] = (float)((int)((i * 2654435761u) >> 20 & 0xfff) - 2048) / 2048.f;
  if (ma) { /* activations and outputs in the pool the context's allocator serves */
    auto place = [&](Tensor &t) {
      void *p = nullptr;
      ma->alloc(&p, mirror_tensor_bytes(t.getDim()), 64);
      t.mirror_move_to(p, [ma](void *q) { ma->free(q); });
    };
    place(b.rc->getInput(0));
    for (unsigned o = 0; o < n_out; ++o)
      place(b.rc->getOutput(o));
  }
  return b;
}

double time_chain(std::vector<BuiltLayer> &chain, bool decode, int iters) {
  auto once = [&]() {
    for (auto &b : chain) {
      if (decode)
        b.layer->incremental_forwarding(*b.rc, 3, 4, false);
      else
        b.layer->incremental_forwarding(*b.rc, 0, b.rc->getInput(0).height(), false);
    }
  };
  for (int i = 0; i < 3; ++i)
    once();
  const auto t0 = std::chrono::steady_clock::now();
  for (int i = 0; i < iters; ++i)
    once();
  const auto t1 = std::chrono::steady_clock::now();
  return std::chrono::duration<double, std::micro>(t1 - t0).count() / iters;
}
} // namespace

static int run_c5layer(Context *ctx, int iters) {
  const unsigned D = 1024, NQ = 2048, NKV = 1024, FF = 3072;
  auto ma = ctx->getContextData() ? ctx->getContextData()->getMemAllocator() : nullptr;
  auto unit = [](unsigned n) { return std::vector<std::string>{"unit=" + std::to_string(n), "disable_bias=true"}; };
  std::printf("{");
  bool first = true, fused_equal = true;
  for (int pinned = 0; pinned < 2; ++pinned) {
    for (int decode = 1; decode >= 0; --decode) {
      const unsigned h = decode ? 8 : 512;
      const auto mem = pinned ? ma : std::shared_ptr<MemAllocator>();
      std::vector<BuiltLayer> seven, four, three;
      seven.push_back(build(ctx, "fully_connected", unit(NQ), h, D, 1, 1, mem));
      seven.push_back(build(ctx, "fully_connected", unit(NKV), h, D, 1, 2, mem));
      seven.push_back(build(ctx, "fully_connected", unit(NKV), h, D, 1, 3, mem));
      seven.push_back(build(ctx, "fully_connected", unit(D), h, NQ, 1, 4, mem));
      seven.push_back(build(ctx, "fully_connected", unit(FF), h, D, 1, 5, mem));
      seven.push_back(build(ctx, "fully_connected", unit(FF), h, D, 1, 6, mem));
      seven.push_back(build(ctx, "fully_connected", unit(D), h, FF, 1, 7, mem));
      four.push_back(build(ctx, "qkv_layer",
                           {"q_unit=" + std::to_string(NQ), "k_unit=" + std::to_string(NKV),
                            "v_unit=" + std::to_string(NKV)},
                           h, D, 3, 11, mem));
      four.push_back(build(ctx, "fully_connected", unit(D), h, NQ, 1, 14, mem));
      four.push_back(build(ctx, "mlp_swiglu", unit(FF), h, D, 1, 15, mem));
      four.push_back(build(ctx, "fully_connected", unit(D), h, FF, 1, 17, mem));
      /* the whole MLP as one layer: the same three weights as four[2] and four[3] */
      std::vector<std::string> mlp_props = unit(FF);
      mlp_props.push_back("down_unit=" + std::to_string(D));
      three.push_back(build(ctx, "qkv_layer",
                            {"q_unit=" + std::to_string(NQ), "k_unit=" + std::to_string(NKV),
                             "v_unit=" + std::to_string(NKV)},
                            h, D, 3, 11, mem));
      three.push_back(build(ctx, "fully_connected", unit(D), h, NQ, 1, 14, mem));
      three.push_back(build(ctx, "mlp_swiglu", mlp_props, h, D, 1, 15, mem));
      const int n = decode ? iters : (iters + 9) / 10;
      const double t7 = time_chain(seven, decode, n), t4 = time_chain(four, decode, n),
                   t3 = time_chain(three, decode, n);
      /* the one-layer MLP against the two layers it replaces, the hidden rows handed over on the host */
      {
        const unsigned rows = decode ? 1 : h;
        std::memcpy(four[3].rc->getInput(0).getData<float>(), four[2].rc->getOutput(0).getData<float>(),
                    (size_t)rows * FF * sizeof(float));
        four[3].layer->incremental_forwarding(*four[3].rc, decode ? 3 : 0, decode ? 4 : h, false);
        if (std::memcmp(four[3].rc->getOutput(0).getData<float>(), three[2].rc->getOutput(0).getData<float>(),
                        (size_t)rows * D * sizeof(float)) != 0)
          fused_equal = false;
      }
      const char *rows_name = decode ? "decode_row" : "prefill_512_rows";
      const char *mem_name = pinned ? "allocator_memory" : "ordinary_memory";
      std::printf("%s\"%s_%s_seven_fully_connected_us\": %.2f, \"%s_%s_qkv_fc_mlp_swiglu_fc_us\": %.2f, "
                  "\"%s_%s_qkv_fc_mlp_us\": %.2f",
                  first ? "" : ", ", rows_name, mem_name, t7, rows_name, mem_name, t4, rows_name, mem_name, t3);
      first = false;
    }
  }
  std::printf(", \"one_layer_mlp_equals_mlp_swiglu_then_fully_connected_bit_for_bit\": %s}\n",
              fused_equal ? "true" : "false");
  return fused_equal ? 0 : 1;
}

static int run_moelayer(Context *ctx, int iters) {
  const unsigned H = 2048, I = 768, E = 128, K = 8;
  auto ma = ctx->getContextData() ? ctx->getContextData()->getMemAllocator() : nullptr;
  std::printf("{");
  bool first = true;
  for (int pinned = 0; pinned < 2; ++pinned) {
    for (unsigned T : {1u, 64u}) {
      auto layer = ctx->createLayerObject("qwen_moe", {"num_experts=" + std::to_string(E),
                                                        "num_experts_per_token=" + std::to_string(K),
                                                        "unit=" + std::to_string(I), "moe_activation=swish"});
      InitLayerContext ic({TensorDim(1, 1, T, H)}, "moe", Tformat::NCHW, Tdatatype::Q4_K, Tdatatype::FP32);
      layer->finalize(ic);
      RunLayerContext rc(ic);
      uint32_t x = 12345u + T;
      float *wr = rc.getWeight(0).getData<float>();
      for (size_t i = 0; i < (size_t)H * E; ++i) {
        x = x * 1664525u + 1013904223u;
        wr[i] = ((int)(x >> 20) - 2048) / 40960.f;
      }
      for (unsigned w = 1; w < rc.getNumWeights(); ++w) {
        /* x8-repacked Q4_K as the tensor holds it: groups of 1152 bytes, eight fp16 scales and eight
         * fp16 mins (2^-8 here), then 96 bytes of 6-bit scales and 1024 of nibbles */
        uint8_t *p = rc.getWeight(w).getData<uint8_t>();
        const size_t bytes = mirror_tensor_bytes(rc.getWeight(w).getDim());
        for (size_t g = 0; g + 1152 <= bytes; g += 1152) {
          for (int i = 0; i < 16; ++i) {
            p[g + 2 * i] = 0x00;
            p[g + 2 * i + 1] = 0x1c;
          }
          for (int i = 32; i < 1152; ++i) {
            x = x * 1664525u + 1013904223u;
            p[g + i] = (uint8_t)(x >> 24);
          }
        }
      }
      float *in = rc.getInput(0).getData<float>();
      for (size_t i = 0; i < (size_t)T * H; ++i)
        in[i] = (float)((int)((i * 2654435761u) >> 20 & 0xfff) - 2048) / 2048.f;
      if (pinned && ma) {
        auto place = [&](Tensor &t) {
          void *q = nullptr;
          ma->alloc(&q, mirror_tensor_bytes(t.getDim()), 64);
          t.mirror_move_to(q, [ma](void *r) { ma->free(r); });
        };
        place(rc.getInput(0));
        place(rc.getOutput(0));
      }
      const int n = T == 1 ? iters : (iters + 3) / 4;
      for (int i = 0; i < 3; ++i)
        layer->incremental_forwarding(rc, 0, T, false);
      const auto t0 = std::chrono::steady_clock::now();
      for (int i = 0; i < n; ++i)
        layer->incremental_forwarding(rc, 0, T, false);
      const auto t1 = std::chrono::steady_clock::now();
      std::printf("%s\"%s_%s_us\": %.2f", first ? "" : ", ", T == 1 ? "decode_token" : "chunk_of_64_tokens",
                  pinned ? "allocator_memory" : "ordinary_memory",
                  std::chrono::duration<double, std::micro>(t1 - t0).count() / n);
      first = false;
    }
  }
  std::printf("}\n");
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 3) {
    std::printf("usage: %s <plugin.so> api | c5layer <iterations> | moelayer <iterations> | fc ... | moe ...\n", argv[0]);
    return 2;
  }
  try {
    Context *ctx = load_context(argv[1]);
    const std::string mode = argv[2];
    if (mode == "c5layer" && argc == 4)
      return run_c5layer(ctx, std::atoi(argv[3]));
    if (mode == "moelayer" && argc == 4)
      return run_moelayer(ctx, std::atoi(argv[3]));
    if (mode == "api")
      return run_api(ctx);
    if (mode == "fc" && argc == 14)
      return run_fc(ctx, argv + 3);
    if (mode == "moe" && (argc == 14 || argc == 16))
      return run_moe(ctx, argv + 3, argc == 16 ? argv + 14 : nullptr);
    if (mode == "fcreload" && argc == 13)
      return run_fc_reload(ctx, argv + 3);
    if (mode == "moex" && argc == 14)
      return run_moex(ctx, argv + 3);
    if (mode == "qkv" && argc == 14)
      return run_qkv(ctx, argv + 3);
    if (mode == "mlp" && (argc == 13 || argc == 14))
      return run_mlp(ctx, argv + 3, argc == 14 ? (unsigned)std::atoi(argv[13]) : 0);
    if ((mode == "lmhead" || mode == "embed") && argc == 13)
      return run_tie(ctx, mode == "lmhead", argv + 3);
    std::printf("bad arguments for mode %s (argc %d)\n", mode.c_str(), argc);
    return 2;
  } catch (const std::exception &e) {
    std::printf("EXCEPTION %s\n", e.what());
    return 3;
  }
}
