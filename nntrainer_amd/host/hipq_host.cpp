// SPDX-License-Identifier: Apache-2.0
/**
 * @file   hipq_host.cpp
 * @brief  Host core of the HIP plug-in: status -> exception translation, the
 *         weight cache and thin typed wrappers over the C ABI (see hipq_host.h).
 */
#include "hipq_host.h"

#include <atomic>
#include <cstring>
#include <sstream>

namespace hipq_host {

void check(int status, const char *what) {
  if (status == HIPQ_OK)
    return;
  std::ostringstream msg;
  const char *detail = hipq_last_error();
  msg << "[hipq] " << what << " failed (" << status << ")";
  if (detail && *detail)
    msg << ": " << detail;
  switch (status) {
  case HIPQ_ERR_INVALID_ARGUMENT:
    throw std::invalid_argument(msg.str());
  case HIPQ_ERR_NOT_SUPPORTED:
    throw not_supported(msg.str());
  case HIPQ_ERR_OUT_OF_MEMORY:
    throw std::bad_alloc();
  default:
    throw std::runtime_error(msg.str());
  }
}

bool runtime_available(int device) noexcept {
  /* 0 = not tried, 1 = up, 2 = unavailable */
  static std::atomic<int> state{0};
  static std::mutex mtx;
  int s = state.load(std::memory_order_acquire);
  if (s)
    return s == 1;
  std::lock_guard<std::mutex> lock(mtx);
  s = state.load(std::memory_order_relaxed);
  if (s)
    return s == 1;
  s = hipq_init(device) == HIPQ_OK ? 1 : 2;
  state.store(s, std::memory_order_release);
  return s == 1;
}

WeightCache::~WeightCache() { clear(); }

/* Eight 8-byte words of the buffer (both ends and six in between) folded into one:
 * cheap enough for every forward call, and a rewritten weight differs in them. */
uint64_t WeightCache::sample(const void *bytes, int64_t n) {
  const unsigned char *p = static_cast<const unsigned char *>(bytes);
  uint64_t tag = 0x9e3779b97f4a7c15ull ^ (uint64_t)n;
  if (n < 8)
    return tag;
  const int64_t last = n - 8;
  for (int i = 0; i < 8; ++i) {
    uint64_t v;
    std::memcpy(&v, p + (last * i / 7), 8);
    tag = (tag ^ v) * 0xff51afd7ed558ccdull;
    tag ^= tag >> 29;
  }
  return tag;
}

hipq_weight_t WeightCache::get(const void *host_bytes, const WeightSpec &spec) {
  if (!host_bytes)
    throw std::invalid_argument("[hipq] weight tensor has no data");
  const int64_t nbytes = hipq_weight_nbytes(spec.dtype, spec.N, spec.K);
  if (nbytes < 0)
    check((int)nbytes, "hipq_weight_nbytes");
  const uint64_t tag = sample(host_bytes, nbytes);
  std::lock_guard<std::mutex> lock(mtx);
  auto it = map.find(host_bytes);
  if (it != map.end()) {
    const WeightSpec &o = it->second.spec;
    if (o.dtype == spec.dtype && o.layout == spec.layout && o.N == spec.N && o.K == spec.K &&
        it->second.tag == tag)
      return it->second.w;
    /* the allocator handed the address to another tensor, or the bytes were rewritten: replace */
    hipq_weight_destroy(it->second.w);
    map.erase(it);
    freed.fetch_add(1, std::memory_order_release);
  }
  hipq_weight_t w = nullptr;
  check(hipq_weight_create(spec.dtype, spec.layout, spec.N, spec.K, host_bytes, HIPQ_MEM_HOST, &w),
        "hipq_weight_create");
  map.emplace(host_bytes, Entry{w, spec, tag});
  return w;
}

void WeightCache::invalidate(const void *host_bytes) {
  std::lock_guard<std::mutex> lock(mtx);
  auto it = map.find(host_bytes);
  if (it == map.end())
    return;
  hipq_weight_destroy(it->second.w);
  map.erase(it);
  freed.fetch_add(1, std::memory_order_release);
}

void WeightCache::clear() {
  std::lock_guard<std::mutex> lock(mtx);
  for (auto &kv : map)
    hipq_weight_destroy(kv.second.w);
  if (!map.empty())
    freed.fetch_add(1, std::memory_order_release);
  map.clear();
}

size_t WeightCache::size() const {
  std::lock_guard<std::mutex> lock(mtx);
  return map.size();
}

WeightCache &global_cache() {
  /* never destroyed: contexts live as long as the process
   * (nntrainer/engine.h:52-57) and the device may be gone at exit */
  static WeightCache *cache = new WeightCache();
  return *cache;
}

static void require_runtime() {
  if (!runtime_available())
    throw std::runtime_error(std::string("[hipq] no usable HIP device: ") + hipq_last_error());
}

void matmul(WeightCache &cache, const void *weight_bytes, const WeightSpec &spec, const float *A,
            int64_t M, int64_t lda, float *C, int64_t ldc) {
  require_runtime();
  hipq_weight_t w = cache.get(weight_bytes, spec);
  check(hipq_matmul(w, A, M, lda, C, ldc, HIPQ_MEM_HOST, nullptr), "hipq_matmul");
}

void matmul_each_row(WeightCache &cache, const void *weight_bytes, const WeightSpec &spec, const float *A,
                     int64_t rows, int64_t lda, float *C, int64_t ldc) {
  require_runtime();
  hipq_weight_t w = cache.get(weight_bytes, spec);
  check(hipq_matmul_each_row(w, A, rows, lda, C, ldc, HIPQ_MEM_HOST, nullptr), "hipq_matmul_each_row");
}

void matmul_multi(WeightCache &cache, const std::vector<const void *> &weight_bytes,
                  const std::vector<WeightSpec> &specs, const float *A, int64_t M, int64_t lda,
                  const std::vector<float *> &C) {
  require_runtime();
  if (weight_bytes.size() != specs.size() || weight_bytes.size() != C.size() || specs.empty())
    throw std::invalid_argument("[hipq] matmul_multi: weights, specs and outputs differ in number");
  std::vector<hipq_weight_t> ws(specs.size());
  std::vector<int64_t> ldc(specs.size());
  for (size_t i = 0; i < specs.size(); ++i) {
    ws[i] = cache.get(weight_bytes[i], specs[i]);
    ldc[i] = specs[i].N;
  }
  check(hipq_matmul_multi((int)ws.size(), ws.data(), A, M, lda, C.data(), ldc.data(), HIPQ_MEM_HOST,
                          nullptr),
        "hipq_matmul_multi");
}

void mlp_swiglu(WeightCache &cache, const void *act_bytes, const void *mul_bytes, const WeightSpec &spec,
                const float *A, int64_t M, int64_t lda, float *out, int64_t ldo) {
  require_runtime();
  hipq_weight_t wa = cache.get(act_bytes, spec), wm = cache.get(mul_bytes, spec);
  check(hipq_mlp_swiglu(wa, wm, A, M, lda, out, ldo, HIPQ_MEM_HOST, nullptr), "hipq_mlp_swiglu");
}

void mlp_swiglu_down(WeightCache &cache, const void *act_bytes, const void *mul_bytes, const WeightSpec &spec,
                     const void *down_bytes, const WeightSpec &down_spec, const float *A, int64_t M, int64_t lda,
                     float *out, int64_t ldo) {
  require_runtime();
  hipq_weight_t wa = cache.get(act_bytes, spec), wm = cache.get(mul_bytes, spec), wd = cache.get(down_bytes, down_spec);
  check(hipq_mlp_swiglu_down(wa, wm, wd, A, M, lda, out, ldo, HIPQ_MEM_HOST, nullptr), "hipq_mlp_swiglu_down");
}

hipq_weight_t upload(const void *host_bytes, const WeightSpec &spec) {
  require_runtime();
  if (!host_bytes)
    throw std::invalid_argument("[hipq] upload: the weight has no bytes (a virtual tensor that is not active?)");
  hipq_weight_t w = nullptr;
  check(hipq_weight_create(spec.dtype, spec.layout, spec.N, spec.K, host_bytes, HIPQ_MEM_HOST, &w),
        "hipq_weight_create");
  return w;
}

float *device_floats(const float *host, size_t n) {
  require_runtime();
  if (!host)
    throw std::invalid_argument("[hipq] device_floats: the tensor has no data");
  void *p = nullptr;
  check(hipq_device_alloc(&p, n * sizeof(float)), "hipq_device_alloc");
  const int rc = hipq_device_upload(p, host, n * sizeof(float), nullptr);
  if (rc != HIPQ_OK) {
    hipq_device_free(p);
    check(rc, "hipq_device_upload");
  }
  return static_cast<float *>(p);
}

void device_release(void *p) noexcept {
  if (p)
    hipq_device_free(p);
}

const float *DeviceMirror::get(const float *host, size_t n) {
  const uint64_t t = WeightCache::sample(host, (int64_t)(n * sizeof(float)));
  if (dev && src == host && count == n && tag == t)
    return dev;
  drop();
  dev = device_floats(host, n);
  src = host;
  count = n;
  tag = t;
  return dev;
}

void DeviceMirror::drop() noexcept {
  device_release(dev);
  dev = nullptr;
}

void release(hipq_weight_t w) noexcept {
  if (w)
    hipq_weight_destroy(w);
}

void moe_forward_resident(const MoeShape &shape, const hipq_weight_t *gate, const hipq_weight_t *up,
                          const hipq_weight_t *down, const float *x, const float *router_weight, float *y,
                          const MoeExtras *extras) {
  require_runtime();
  hipq_moe_desc desc;
  desc.tokens = shape.tokens;
  desc.hidden = shape.hidden;
  desc.intermediate = shape.intermediate;
  desc.experts = shape.experts;
  desc.topk = shape.topk;
  desc.renormalize = shape.renormalize ? 1 : 0;
  hipq_moe_ext ext;
  ext.variant = extras && extras->gpt_oss ? HIPQ_MOE_GPT_OSS : HIPQ_MOE_QWEN;
  ext.alpha = extras ? extras->alpha : 0.f;
  ext.router_bias = extras ? extras->router_bias : nullptr;
  ext.gate_bias = extras ? extras->gate_bias : nullptr;
  ext.up_bias = extras ? extras->up_bias : nullptr;
  ext.down_bias = extras ? extras->down_bias : nullptr;
  ext.limit = extras ? extras->limit : 0.f;
  ext.biases_on_device = extras && extras->biases_on_device ? 1 : 0;
  ext.router_on_device = extras && extras->router_on_device ? 1 : 0;
  check(hipq_moe_forward_ext(&desc, &ext, gate, up, down, x, nullptr, router_weight, y, nullptr, nullptr,
                             HIPQ_MEM_HOST, nullptr),
        "hipq_moe_forward");
}

void moe_forward(WeightCache &cache, const MoeShape &shape, int dtype,
                 const std::vector<const void *> &gate_bytes,
                 const std::vector<const void *> &up_bytes,
                 const std::vector<const void *> &down_bytes, const float *x,
                 const float *router_weight, float *y, const MoeExtras *extras, HandleMemo *memo) {
  require_runtime();
  const size_t E = (size_t)shape.experts;
  if (gate_bytes.size() != E || up_bytes.size() != E || down_bytes.size() != E)
    throw std::invalid_argument("[hipq] moe_forward: one gate, up and down weight per expert");
  const int layout = framework_layout(dtype);
  const WeightSpec gu{dtype, layout, shape.intermediate, shape.hidden};
  const WeightSpec dn{dtype, layout, shape.hidden, shape.intermediate};
  HandleMemo local;
  HandleMemo &m = memo ? *memo : local;
  /* gate, up and down handles in one array: [0, E), [E, 2E), [2E, 3E) */
  const bool known = m.w.size() == 3 * E && m.epoch == cache.epoch();
  if (!known) {
    m.bytes.assign(3 * E, nullptr);
    m.tags.assign(3 * E, 0);
    m.w.assign(3 * E, nullptr);
  }
  const int64_t nb_gu = hipq_weight_nbytes(gu.dtype, gu.N, gu.K), nb_dn = hipq_weight_nbytes(dn.dtype, dn.N, dn.K);
  bool replaced = false;
  auto resolve = [&](size_t i, const void *bytes, const WeightSpec &spec, int64_t nbytes) {
    if (!bytes)
      throw std::invalid_argument("[hipq] weight tensor has no data");
    const uint64_t tag = nbytes >= 0 ? WeightCache::sample(bytes, nbytes) : 0;
    if (known && m.bytes[i] == bytes && m.tags[i] == tag)
      return; /* the tensor of the last call, unchanged: its handle stands */
    const uint64_t before = cache.epoch();
    m.w[i] = cache.get(bytes, spec);
    replaced |= cache.epoch() != before;
    m.bytes[i] = bytes;
    m.tags[i] = tag;
  };
  for (size_t e = 0; e < E; ++e) {
    resolve(e, gate_bytes[e], gu, nb_gu);
    resolve(E + e, up_bytes[e], gu, nb_gu);
    resolve(2 * E + e, down_bytes[e], dn, nb_dn);
  }
  /* a replacement freed a device copy: handles resolved before it in this call may be that copy */
  if (replaced)
    for (size_t e = 0; e < E; ++e) {
      m.w[e] = cache.get(gate_bytes[e], gu);
      m.w[E + e] = cache.get(up_bytes[e], gu);
      m.w[2 * E + e] = cache.get(down_bytes[e], dn);
    }
  m.epoch = cache.epoch();
  moe_forward_resident(shape, m.w.data(), m.w.data() + E, m.w.data() + 2 * E, x, router_weight, y, extras);
}

} // namespace hipq_host
