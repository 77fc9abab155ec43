// SPDX-License-Identifier: Apache-2.0
/**
 * @file   nntr_api_mirror.h
 * @brief  Stand-in for the part of the framework's plug-in API that the HIP
 *         context and its layers touch, for builds outside the framework's tree.
 *
 * Inside the framework the adapters include the real headers (define
 * HIPQ_WITH_NNTRAINER). Here every class keeps the name, the member names and
 * the argument meaning of its original so that the adapter sources compile
 * unchanged against either:
 *   Context, ContextData, ContextPluggable   nntrainer/context.h:31-240
 *   Layer, createLayer                        nntrainer/layers/layer_devel.h:81-508
 *   InitLayerContext, RunLayerContext         nntrainer/layers/layer_context.h:42-430, 460-1010
 *   TensorDim                                 api/ccapi/include/tensor_dim.h:40-330
 *   Tensor                                    nntrainer/tensor/tensor.h
 *   exception::not_supported, NNTR_THROW_IF   nntrainer/nntrainer_error.h:32-34, 157-159
 * Only what this path uses is present; the bodies are written for this stand-in
 * (host memory owned by std::vector) and carry none of the framework's logic.
 */
#ifndef NNTR_API_MIRROR_H
#define NNTR_API_MIRROR_H

#include <array>
#include <bitset>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <functional>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <tuple>
#include <unordered_map>
#include <variant>
#include <vector>

namespace ml {
namespace train {

/** integer keys of layer types; only the one this plug-in registers */
enum LayerType { LAYER_FC = 1 };

enum class ExportMethods { METHOD_STRINGVECTOR = 0 };
enum class ExecutionMode { TRAIN = 0, INFERENCE = 1 };

class TensorDim {
public:
  enum class Format { NCHW, NHWC };
  enum class DataType { QINT4, QINT8, QINT16, BCQ, Q4_K, Q6_K, Q4_0, UINT8, UINT16, UINT32, FP16, FP32 };

  struct TensorType {
    Format format;
    DataType data_type;
    TensorType() : format(Format::NCHW), data_type(DataType::FP32) {}
    TensorType(Format fm, DataType dt) : format(fm), data_type(dt) {}
  };

  explicit TensorDim(TensorType t = TensorType()) : t_type(t) { dim = {0, 0, 0, 0}; }
  TensorDim(size_t b, size_t c, size_t h, size_t w, TensorType t = TensorType(),
            const std::bitset<4> & /*eff_dim_flag*/ = 0b1111) :
    t_type(t) {
    dim = {b, c, h, w};
  }
  TensorDim(std::initializer_list<size_t> dims, TensorType t = TensorType()) : t_type(t) {
    dim = {1, 1, 1, 1};
    size_t i = 4 - dims.size();
    for (size_t d : dims)
      dim[i++] = d;
  }

  size_t batch() const { return dim[0]; }
  size_t channel() const { return dim[1]; }
  size_t height() const { return dim[2]; }
  size_t width() const { return dim[3]; }
  void batch(size_t b) { dim[0] = b; }
  void channel(size_t c) { dim[1] = c; }
  void height(size_t h) { dim[2] = h; }
  void width(size_t w) { dim[3] = w; }
  size_t getFeatureLen() const { return dim[1] * dim[2] * dim[3]; }
  size_t getDataLen() const { return dim[0] * getFeatureLen(); }
  DataType getDataType() const { return t_type.data_type; }
  Format getFormat() const { return t_type.format; }
  void setDataType(DataType d) { t_type.data_type = d; }
  void setTensorType(TensorType t) { t_type = t; }
  TensorType getTensorType() const { return t_type; }
  bool operator==(const TensorDim &o) const { return dim == o.dim; }

private:
  std::array<size_t, 4> dim;
  TensorType t_type;
};

} // namespace train
} // namespace ml

namespace nntrainer {

using TensorDim = ml::train::TensorDim;
using Tformat = ml::train::TensorDim::Format;
using Tdatatype = ml::train::TensorDim::DataType;

enum class Initializer { ZEROS, ONES, NONE };
enum class WeightRegularizer { L2NORM, NONE, UNKNOWN };
enum class TensorLifespan { FORWARD_FUNC_LIFESPAN, MAX_LIFESPAN };

namespace exception {
struct not_supported : public std::invalid_argument {
  using invalid_argument::invalid_argument;
};
/** collects a message with << and throws when it goes out of scope */
template <typename Err> struct ErrorNotification {
  std::ostringstream ss;
  ErrorNotification() = default;
  [[noreturn]] ~ErrorNotification() noexcept(false) { throw Err(ss.str()); }
  template <typename T> ErrorNotification &operator<<(const T &v) {
    ss << v;
    return *this;
  }
};
} // namespace exception

#define NNTR_THROW_IF(pred, err) \
  if ((pred))                    \
  nntrainer::exception::ErrorNotification<err> {}

/** bytes of a tensor of quantized blocks or plain elements */
inline size_t mirror_tensor_bytes(const TensorDim &d) {
  const size_t n = d.getDataLen();
  switch (d.getDataType()) {
  case Tdatatype::Q4_0:
    return n / 32 * 18;
  case Tdatatype::Q4_K:
    return n / 256 * 144;
  case Tdatatype::Q6_K:
    return n / 256 * 210;
  case Tdatatype::FP16:
  case Tdatatype::UINT16:
    return n * 2;
  case Tdatatype::UINT8:
  case Tdatatype::QINT8:
    return n;
  default:
    return n * 4;
  }
}

/** where a layer's weights are read from (nntrainer/utils/util_func.h:43) */
using ReadSource = std::variant<std::ifstream *, const char *>;

/** The bytes of a tensor: the stand-in's own memory, or memory that a driver took from a
 *  MemAllocator, as the framework hands a context's allocator to its memory pool (engine.h:82-84,
 *  tensor/memory_pool.h:110). */
class MirrorBytes {
public:
  explicit MirrorBytes(size_t n) : own(n), p(own.data()), n(n) {}
  explicit MirrorBytes(const std::vector<uint8_t> &v) : own(v), p(own.data()), n(own.size()) {}
  MirrorBytes(void *external, size_t n, std::function<void(void *)> release) :
    p(static_cast<uint8_t *>(external)), n(n), release(std::move(release)) {}
  MirrorBytes(const MirrorBytes &) = delete;
  MirrorBytes &operator=(const MirrorBytes &) = delete;
  ~MirrorBytes() {
    if (release)
      release(p);
  }
  uint8_t *data() { return p; }
  size_t size() const { return n; }

private:
  std::vector<uint8_t> own;
  uint8_t *p;
  size_t n;
  std::function<void(void *)> release;
};

/** Host tensor: a view (offset + dims) into shared storage. */
class Tensor {
public:
  /** the tensor's bytes from a model file, in place (tensor.h:1646-1655) */
  void read(std::ifstream &file, size_t start_offset = 0, bool read_from_offset = false, int /*file_fd*/ = -1) {
    if (read_from_offset)
      file.seekg((std::streamoff)start_offset);
    /* a virtual tensor only notes where its bytes are (tensor.cpp, read of a virtual tensor) */
    char *dst = is_virtual ? reinterpret_cast<char *>(this->file->data()) : getData<char>();
    file.read(dst, (std::streamsize)mirror_tensor_bytes(dim));
    NNTR_THROW_IF(file.fail(), std::runtime_error) << "short read of a tensor";
  }
  void read(ReadSource src, size_t start_offset = 0, bool read_from_offset = false) {
    NNTR_THROW_IF(!std::holds_alternative<std::ifstream *>(src), std::invalid_argument) << "file sources only";
    read(*std::get<std::ifstream *>(src), start_offset, read_from_offset);
  }

  Tensor() = default;
  explicit Tensor(const TensorDim &d) : dim(d), store(std::make_shared<MirrorBytes>(mirror_tensor_bytes(d))) {}
  /** moves the tensor's bytes into `external` (of at least its size), released through `release` with the last view */
  void mirror_move_to(void *external, std::function<void(void *)> release) {
    const size_t n = mirror_tensor_bytes(dim);
    if (store)
      std::memcpy(external, getData<uint8_t>(), n);
    store = std::make_shared<MirrorBytes>(external, n, std::move(release));
    offset_bytes = 0;
  }
  /** a virtual tensor (requestWeight(..., is_virtual = true)): its bytes live in the model file
   *  until activate() maps them in and are gone again after deactivate() (tensor.h:1979-1993).
   *  Here the "file" is a second buffer that a test fills through mirror_file_bytes(). */
  static Tensor make_virtual(const TensorDim &d) {
    Tensor t;
    t.dim = d;
    t.is_virtual = true;
    t.file = std::make_shared<std::vector<uint8_t>>(mirror_tensor_bytes(d));
    return t;
  }
  void activate() {
    if (is_virtual && !store)
      store = std::make_shared<MirrorBytes>(*file);
  }
  void deactivate() {
    if (is_virtual)
      store.reset();
  }
  uint8_t *mirror_file_bytes() { return file ? file->data() : nullptr; }
  Tensor(size_t b, size_t c, size_t h, size_t w, TensorDim::TensorType t = TensorDim::TensorType()) :
    Tensor(TensorDim(b, c, h, w, t)) {}

  TensorDim getDim() const { return dim; }
  size_t batch() const { return dim.batch(); }
  size_t channel() const { return dim.channel(); }
  size_t height() const { return dim.height(); }
  size_t width() const { return dim.width(); }
  size_t size() const { return dim.getDataLen(); }
  Tdatatype getDataType() const { return dim.getDataType(); }
  TensorDim::TensorType getTensorType() const { return dim.getTensorType(); }
  bool empty() const { return !store; }

  template <typename T = float> T *getData() const {
    return store ? reinterpret_cast<T *>(store->data() + offset_bytes) : nullptr;
  }

  /** a tensor of shape d that shares this tensor's memory from element `offset` on */
  Tensor getSharedDataTensor(const TensorDim &d, size_t offset, bool /*reset_stride*/ = true) const {
    Tensor t;
    t.dim = d;
    t.store = store;
    t.offset_bytes = offset_bytes + offset * 4; /* only fp32 tensors are viewed on this path */
    if (t.offset_bytes + mirror_tensor_bytes(d) > store->size())
      throw std::invalid_argument("shared tensor does not fit its source");
    return t;
  }

  void reshape(const TensorDim &d) {
    if (d.getDataLen() != dim.getDataLen())
      throw std::invalid_argument("reshape changes the number of elements");
    const auto t = dim.getTensorType();
    dim = d;
    dim.setTensorType(t);
  }

  void setZero() {
    if (store)
      std::memset(getData<uint8_t>(), 0, mirror_tensor_bytes(dim));
  }

  /** this += m, with m broadcast over leading dimensions (bias add) */
  int add_i(const Tensor &m, float alpha = 1.f) {
    float *a = getData<float>();
    const float *b = m.getData<float>();
    const size_t n = size(), nb = m.size();
    if (!nb || n % nb)
      throw std::invalid_argument("add_i: operand does not broadcast");
    for (size_t i = 0; i < n; ++i)
      a[i] += alpha * b[i % nb];
    return 0;
  }

private:
  TensorDim dim;
  std::shared_ptr<MirrorBytes> store;
  size_t offset_bytes = 0;
  bool is_virtual = false;
  std::shared_ptr<std::vector<uint8_t>> file;
};

/** What a layer declares in finalize(): weights and scratch tensors by spec. */
class InitLayerContext {
public:
  struct WeightRequest {
    TensorDim dim;
    std::string name;
    bool trainable;
    bool is_virtual;
  };
  struct TensorRequest {
    TensorDim dim;
    std::string name;
  };

  InitLayerContext(const std::vector<TensorDim> &dims, const std::string &name, Tformat fm,
                   Tdatatype weight_type, Tdatatype act_type) :
    input_dims(dims), prefix(name), format(fm), wtype(weight_type), atype(act_type) {}

  unsigned int getNumInputs() const { return input_dims.size(); }
  const std::vector<TensorDim> &getInputDimensions() const { return input_dims; }
  void setOutputDimensions(const std::vector<TensorDim> &d) { output_dims = d; }
  const std::vector<TensorDim> &getOutputDimensions() const { return output_dims; }
  Tformat getFormat() const { return format; }
  Tdatatype getWeightDataType() const { return wtype; }
  Tdatatype getActivationDataType() const { return atype; }
  void setEffDimFlagInputDimension(unsigned int, int) {}
  void setDynDimFlagInputDimension(unsigned int, int) {}
  const std::string &getName() const { return prefix; }

  unsigned int requestWeight(const TensorDim &dim, const Initializer, const WeightRegularizer,
                             const float, const float, const std::string &name, bool trainable = true,
                             bool is_virtual = false, unsigned int = 3) {
    weights.push_back({dim, prefix + ":" + name, trainable, is_virtual});
    return weights.size() - 1;
  }
  unsigned int requestTensor(const TensorDim &dim, const std::string &name,
                             const Initializer = Initializer::NONE, bool = false,
                             TensorLifespan = TensorLifespan::FORWARD_FUNC_LIFESPAN, bool = true) {
    tensors.push_back({dim, prefix + ":" + name});
    return tensors.size() - 1;
  }

  const std::vector<WeightRequest> &getWeightRequests() const { return weights; }
  const std::vector<TensorRequest> &getTensorRequests() const { return tensors; }

private:
  std::vector<TensorDim> input_dims, output_dims;
  std::string prefix;
  Tformat format;
  Tdatatype wtype, atype;
  std::vector<WeightRequest> weights;
  std::vector<TensorRequest> tensors;
};

/** What a layer sees at run time: its inputs, outputs, weights and tensors. */
class RunLayerContext {
public:
  RunLayerContext() = default;
  /** allocates everything a finalized layer asked for */
  explicit RunLayerContext(const InitLayerContext &init) : name(init.getName()) {
    for (auto &d : init.getInputDimensions())
      inputs.emplace_back(d);
    for (auto &d : init.getOutputDimensions())
      outputs.emplace_back(d);
    for (auto &w : init.getWeightRequests())
      weights.push_back(w.is_virtual ? Tensor::make_virtual(w.dim) : Tensor(w.dim));
    for (auto &t : init.getTensorRequests())
      tensors.emplace_back(t.dim);
  }

  Tensor &getInput(unsigned int i) { return inputs.at(i); }
  Tensor &getOutput(unsigned int i) { return outputs.at(i); }
  Tensor &getWeight(unsigned int i) const { return const_cast<Tensor &>(weights.at(i)); }
  Tensor &getTensor(unsigned int i) { return tensors.at(i); }
  unsigned int getNumWeights() const { return weights.size(); }
  const std::string &getName() const { return name; }

private:
  std::string name;
  std::vector<Tensor> inputs, outputs, weights, tensors;
};

class Exporter;

class Layer {
public:
  virtual ~Layer() = default;
  virtual const std::string getType() const = 0;
  virtual void finalize(InitLayerContext &context) = 0;
  virtual void initialize(RunLayerContext &) {}
  virtual void forwarding(RunLayerContext &context, bool training) = 0;
  virtual void incremental_forwarding(RunLayerContext &context, unsigned int, unsigned int, bool training) {
    forwarding(context, training);
  }
  virtual void calcDerivative(RunLayerContext &context) = 0;
  virtual void calcGradient(RunLayerContext &) {}
  virtual void setProperty(const std::vector<std::string> &values) = 0;
  virtual void exportTo(Exporter &, const ml::train::ExportMethods &) const {}
  /** weights from a model file (layer_devel.h:391-470, the inference branch) */
  virtual void read(std::ifstream &file, RunLayerContext &run_context, bool /*opt_var*/,
                    ml::train::ExecutionMode /*mode*/, bool /*trainable*/, TensorDim::DataType /*defineWeightDataType*/,
                    bool /*fsu*/, size_t start_offset = 0, bool read_from_offset = false, int file_fd = -1) {
    for (unsigned int i = 0; i < run_context.getNumWeights(); ++i)
      run_context.getWeight(i).read(file, start_offset, read_from_offset, file_fd);
  }
  virtual void read(ReadSource src, RunLayerContext &run_context, bool /*opt_var*/, ml::train::ExecutionMode /*mode*/,
                    bool /*trainable*/, TensorDim::DataType /*defineWeightDataType*/, bool /*fsu*/,
                    size_t start_offset = 0, bool read_from_offset = false) {
    for (unsigned int i = 0; i < run_context.getNumWeights(); ++i)
      run_context.getWeight(i).read(src, start_offset, read_from_offset);
  }
  virtual void setBatch(RunLayerContext &, unsigned int) {}
  virtual bool supportBackwarding() const = 0;
};

template <typename T, std::enable_if_t<std::is_base_of<Layer, T>::value, T> * = nullptr>
std::unique_ptr<Layer> createLayer(const std::vector<std::string> &props = {}) {
  std::unique_ptr<Layer> ptr = std::make_unique<T>();
  ptr->setProperty(props);
  return ptr;
}

/** nntrainer/mem_allocator.h:24-33, mem_allocator.cpp:22-30 */
class MemAllocator {
public:
  MemAllocator() = default;
  virtual ~MemAllocator() = default;
  virtual void alloc(void **ptr, size_t size, size_t /*alignment*/) { *ptr = std::calloc(size, 1); }
  virtual void free(void *ptr) { std::free(ptr); }
  virtual std::string getName() { return "cpu"; }
};

class ContextData {
public:
  std::shared_ptr<MemAllocator> getMemAllocator() { return mem_allocator; }
  void setMemAllocator(std::shared_ptr<MemAllocator> m) { mem_allocator = m; }

private:
  std::shared_ptr<MemAllocator> mem_allocator;
};

class Context {
public:
  using PropsType = std::vector<std::string>;
  template <typename T> using PtrType = std::unique_ptr<T>;
  template <typename T> using FactoryType = std::function<PtrType<T>(const PropsType &)>;
  template <typename T> using PtrFactoryType = PtrType<T> (*)(const PropsType &);
  template <typename T> using StrIndexType = std::unordered_map<std::string, FactoryType<T>>;
  using IntIndexType = std::unordered_map<int, std::string>;
  template <typename T> using IndexType = std::tuple<StrIndexType<T>, IntIndexType>;
  template <typename... Ts> using FactoryMap = std::tuple<IndexType<Ts>...>;

  Context(std::shared_ptr<ContextData> data_ = nullptr) : data(data_) {}
  virtual ~Context() = default;
  virtual int init() { return 0; }
  virtual PtrType<nntrainer::Layer> createLayerObject(const std::string &, const std::vector<std::string> & = {}) {
    return nullptr;
  }
  virtual PtrType<nntrainer::Layer> createLayerObject(const int, const std::vector<std::string> & = {}) {
    return nullptr;
  }
  virtual std::string getName() = 0;
  std::shared_ptr<ContextData> getContextData() { return data; }
  std::shared_ptr<MemAllocator> getMemAllocator() { return getContextData()->getMemAllocator(); }
  virtual int load(const std::string &) { return 0; }

private:
  std::shared_ptr<ContextData> data;
};

using CreateContextFunc = nntrainer::Context *(*)();
using DestroyContextFunc = void (*)(nntrainer::Context *);
typedef struct {
  CreateContextFunc createfunc;
  DestroyContextFunc destroyfunc;
} ContextPluggable;

} // namespace nntrainer

#endif /* NNTR_API_MIRROR_H */
