// SPDX-License-Identifier: Apache-2.0
/**
 * @file   api.hip
 * @brief  C ABI of libhipq (include/hipq.h): library state, per-stream
 *         workspaces, weight upload, and the matmul / quantize / MoE dispatch.
 *
 * The dispatch in hipq_matmul restates the control flow of the reference
 * wrappers (nntrainer/tensor/cpu_backend/ggml_interface/ggml_interface_omp.cpp:
 * 303-390 Q4_0, 404-487 Q4_K, 500-566 Q6_K in the reference checkout):
 * which activation quantizer each row gets (Q8_0; Q8_K row semantics for M == 1,
 * for the M % 4 leftover rows and for every Q6_K row; Q8_K 4-row semantics for
 * rows [0, 4*(M/4)) of a Q4_K matmul with M > 1), then GEMV for decode shapes
 * and the matrix-core GEMM for prefill shapes. There is no CPU fallback: without
 * a gfx950 device hipq_init fails and every other call reports
 * HIPQ_ERR_NOT_INITIALIZED.
 */
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "hipq_internal.h"

/* Scratch of hipq_matmul_noalloc: quantized activations (and partial products) of one call.
 * Four slots, one per stream that uses the entry point, so that calls on different streams
 * do not share memory. Every GPU the library runs on holds its own copy of the array at its
 * own address until the process ends; in host code the array's name is only a stand-in, the
 * address comes from hipGetSymbolAddress with that device current (hipq_init). */
constexpr int NOALLOC_SLOTS = 4;
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)8 << 20; /* one slot: the most one call may need */
constexpr int MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SLOTS * NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char tl_error[768] = "";

struct Workspace {
  void *ptr = nullptr;
  size_t bytes = 0;
  /* Blocks a call outgrew. They are not freed where they are replaced: kernels already queued
   * read them, and the call that asked may still hold pointers into them. They go when a later
   * call on the stream starts (after the stream has drained) or the stream is released. */
  std::vector<void *> retired;
  int depth = 0;           /* public entry points active on this stream (they nest) */
  uint64_t generation = 0; /* counts the times ptr has changed */
  /* device copies of a host-memory call's operands (the kernels' own scratch is ptr) */
  void *io = nullptr;
  size_t io_bytes = 0;
  /* page-locked staging of a decode step's pageable operands (DirectIO) */
  void *pin = nullptr;
  size_t pin_bytes = 0;
  /* a page-locked word the last launch of such a call writes and the host polls */
  uint32_t *done = nullptr;
  uint32_t done_seq = 0;
  /* a second stream and an event: a prefill's finished rows go back to page-locked host memory on it
   * while the kernels work on the following rows (RowSteps) */
  hipStream_t copy = nullptr;
  hipEvent_t step_done = nullptr;
  /* held while a call enqueues its launches: two threads that name the same stream
   * must not interleave their kernels (the second would quantize into the scratch
   * the first one's product has not read yet) */
  std::recursive_mutex enqueue;
};

struct MoeTable {
  std::vector<const hipq_weight *> key;
  WView *dev = nullptr;
};

struct State {
  std::mutex mu;
  bool ready = false;
  int device = -1;
  void *scratch_ptr[MAX_DEVICES] = {}; /* device address of `scratch`, per device */
  std::recursive_mutex noalloc_enqueue; /* calls of the allocation-free entry point submit one at a time */
  hipStream_t noalloc_stream[NOALLOC_SLOTS] = {}; /* which stream owns which slot of `scratch` */
  bool noalloc_taken[NOALLOC_SLOTS] = {};
  std::unordered_map<hipStream_t, Workspace> ws;
  /* one table of expert weight views per MoE layer, found by its first gate weight */
  std::unordered_map<const hipq_weight *, MoeTable> moe_tables;
  /* held from the look-up of an expert table until the launches that read it are enqueued,
   * and by whoever frees a table: taken before mu, never the other way round */
  std::mutex moe_mu;
  int64_t live_weights = 0;
};
State g;

} // namespace

namespace hipq {
thread_local LaunchLog launch_log;

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tl_error, sizeof(tl_error), fmt, ap);
  va_end(ap);
  return code;
}

} // namespace hipq

using hipq::fail;

namespace {

int require_ready() {
  if (!g.ready) return fail(HIPQ_ERR_NOT_INITIALIZED, "hipq_init has not succeeded");
  hipError_t e = hipSetDevice(g.device);
  if (e != hipSuccess) return fail(HIPQ_ERR_RUNTIME, "hipSetDevice(%d): %s", g.device, hipGetErrorString(e));
  return HIPQ_OK;
}

/* Per-stream scratch, grown on demand. Work queued on one stream runs in order,
 * so consecutive calls on a stream may share it; different streams never do.
 * A request the block cannot serve gets a new block; the old one is retired, not freed, so
 * nothing that was carved out of it earlier in the same call (or is read by kernels already
 * queued) loses its memory. What a larger block does not carry over is the old block's
 * CONTENTS: a call that shares quantized activations between several products reserves the
 * largest request first (one reservation per entry point) and checks workspace_generation()
 * before it reuses them. */
int workspace(hipStream_t s, size_t bytes, void **out) {
  std::lock_guard<std::mutex> lk(g.mu);
  Workspace &w = g.ws[s];
  if (w.bytes < bytes) {
    size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    void *fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, want);
    if (e != hipSuccess)
      return fail(HIPQ_ERR_OUT_OF_MEMORY, "workspace of %zu bytes: %s", want, hipGetErrorString(e));
    if (w.ptr) w.retired.push_back(w.ptr);
    w.ptr = fresh;
    w.bytes = want;
    ++w.generation;
  }
  *out = w.ptr;
  return HIPQ_OK;
}

uint64_t workspace_generation(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g.mu);
  return g.ws[s].generation;
}

/* A call that reuses activations it quantized earlier names the generation it saw then. */
int workspace_unmoved(hipStream_t s, uint64_t generation) {
  if (workspace_generation(s) == generation) return HIPQ_OK;
  return fail(HIPQ_ERR_RUNTIME,
              "internal: the stream's workspace was replaced between the quantization of a call's shared "
              "activations and a product that reads them (a request larger than the call's reservation)");
}

/* Marks a public entry point's stay on a stream. The outermost one frees the blocks earlier
 * calls retired, once the stream has drained -- unless the stream is being captured into a
 * graph, where nothing may wait; they then stay until a later call. */
struct CallScope {
  hipStream_t s;
  explicit CallScope(hipStream_t s_) : s(s_) {
    std::lock_guard<std::mutex> lk(g.mu);
    Workspace &w = g.ws[s];
    if (w.depth++ == 0 && !w.retired.empty()) {
      hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
      if (hipStreamIsCapturing(s, &cs) != hipSuccess) (void)hipGetLastError();
      if (cs == hipStreamCaptureStatusNone && hipStreamSynchronize(s) == hipSuccess) {
        for (void *p : w.retired) (void)hipFree(p);
        w.retired.clear();
      }
    }
  }
  ~CallScope() {
    std::lock_guard<std::mutex> lk(g.mu);
    --g.ws[s].depth;
  }
  CallScope(const CallScope &) = delete;
  CallScope &operator=(const CallScope &) = delete;
};

int io_buffer(hipStream_t s, size_t bytes, void **out) {
  std::lock_guard<std::mutex> lk(g.mu);
  Workspace &w = g.ws[s];
  if (w.io_bytes < bytes) {
    if (w.io) {
      HIPQ_HIP(hipStreamSynchronize(s));
      HIPQ_HIP(hipFree(w.io));
      w.io = nullptr;
      w.io_bytes = 0;
    }
    size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    hipError_t e = hipMalloc(&w.io, want);
    if (e != hipSuccess) {
      w.io = nullptr;
      return fail(HIPQ_ERR_OUT_OF_MEMORY, "operand buffer of %zu bytes: %s", want, hipGetErrorString(e));
    }
    w.io_bytes = want;
  }
  *out = w.io;
  return HIPQ_OK;
}

/* Host memory the framework hands over is pageable: a copy from it goes through the runtime's
 * own small staging and reaches a few GB/s. This ring of pinned slots takes its place: the
 * caller's thread copies a slice into a slot while the DMA engine moves the slice before it, so
 * a transfer runs at the speed of a host memcpy. Memory that is pinned already (the allocator of
 * hipq_host_alloc, or any hipHostMalloc) is handed to the DMA engine as it is. One ring per
 * process, one transfer at a time; a slot is reused once the event recorded behind its last
 * copy has passed, whichever stream that copy was on. */
struct StageRing {
  static constexpr int SLOTS = 4;
  static constexpr size_t SLOT_BYTES = (size_t)2 << 20;
  std::mutex mu;
  char *base = nullptr;
  hipEvent_t ev[SLOTS];
  bool busy[SLOTS] = {false, false, false, false}; /* ev[k] was recorded after the slot's last use */
  size_t pos = 0;                                  /* slots are taken round robin across transfers */
  /* the slot is free again: the copy that read or wrote it last has completed */
  int wait_free(int k) {
    if (busy[k]) {
      HIPQ_HIP(hipEventSynchronize(ev[k]));
      busy[k] = false;
    }
    return HIPQ_OK;
  }
  int ensure() {
    if (base) return HIPQ_OK;
    HIPQ_HIP(hipHostMalloc((void **)&base, SLOTS * SLOT_BYTES, hipHostMallocDefault));
    for (int i = 0; i < SLOTS; ++i) HIPQ_HIP(hipEventCreateWithFlags(&ev[i], hipEventDisableTiming));
    return HIPQ_OK;
  }
};
StageRing g_ring;

bool is_pinned(const void *p) {
  hipPointerAttribute_t at;
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError(); /* an ordinary host pointer: not an error of ours */
    return false;
  }
  return at.type == hipMemoryTypeHost;
}

/* The address the GPU uses for page-locked host memory (null if p is none). */
void *pinned_device_ptr(const void *p) {
  hipPointerAttribute_t at;
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (at.type != hipMemoryTypeHost) return nullptr;
  void *d = nullptr;
  if (hipHostGetDevicePointer(&d, const_cast<void *>(p), 0) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  return d;
}

/* A few rows of page-locked host memory into a dense device buffer, by a kernel: each value
 * crosses the bus once, and a launch costs less than a copy engine's start. */
__global__ __launch_bounds__(256) void fetch_rows_kernel(const float *__restrict__ src, int64_t lds, float *__restrict__ dst,
                                                         int K, int rows) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= (int64_t)rows * K) return;
  const int r = (int)(i / K), c = (int)(i - (int64_t)r * K); /* K % 4 == 0 */
  *(float4 *)(dst + i) = *(const float4 *)(src + r * lds + c);
}

/* The stream's page-locked staging buffer, grown on demand (the stream is idle when it grows: the
 * calls that use it are synchronous and hold the stream's enqueue lock). */
int pinned_staging(hipStream_t s, size_t bytes, void **out) {
  std::lock_guard<std::mutex> lk(g.mu);
  Workspace &w = g.ws[s];
  if (w.pin_bytes < bytes) {
    if (w.pin) {
      HIPQ_HIP(hipStreamSynchronize(s));
      HIPQ_HIP(hipHostFree(w.pin));
      w.pin = nullptr;
      w.pin_bytes = 0;
    }
    const size_t want = (bytes + ((size_t)1 << 16) - 1) & ~(((size_t)1 << 16) - 1);
    hipError_t e = hipHostMalloc(&w.pin, want, hipHostMallocDefault);
    if (e != hipSuccess) {
      w.pin = nullptr;
      return fail(HIPQ_ERR_OUT_OF_MEMORY, "page-locked staging of %zu bytes: %s", want, hipGetErrorString(e));
    }
    w.pin_bytes = want;
  }
  *out = w.pin;
  return HIPQ_OK;
}

/* The end of a short synchronous call: a one-thread kernel behind the call's launches writes the
 * call's number into a page-locked word and the host polls that word. Waking a thread out of
 * hipStreamSynchronize costs several microseconds more than the poll sees the store; a call that
 * takes longer than the poll is patient falls back to the stream's wait. */
__global__ void signal_done_kernel(uint32_t *word, uint32_t value) {
  __hip_atomic_store(word, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}
int wait_done(hipStream_t s) {
  uint32_t *word = nullptr, seq = 0;
  {
    std::lock_guard<std::mutex> lk(g.mu);
    Workspace &w = g.ws[s];
    if (!w.done) {
      hipError_t e = hipHostMalloc((void **)&w.done, 64, hipHostMallocDefault);
      if (e != hipSuccess) {
        w.done = nullptr;
        (void)hipGetLastError();
      } else
        *w.done = 0;
    }
    word = w.done;
    seq = ++w.done_seq;
  }
  if (!word) {
    HIPQ_HIP(hipStreamSynchronize(s));
    return HIPQ_OK;
  }
  hipq::launch_kernel("signal_done_kernel", signal_done_kernel, dim3(1), dim3(1), 0, s, (uint32_t *)pinned_device_ptr(word), seq);
  HIPQ_HIP(hipGetLastError());
  for (int spin = 0; spin < 200000; ++spin) { /* about a tenth of a millisecond */
    if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == seq) return HIPQ_OK;
    __builtin_ia32_pause();
  }
  HIPQ_HIP(hipStreamSynchronize(s));
  return HIPQ_OK;
}

/* A few rows of host operands without a copy engine. Up to 128 rows and 2 MiB a side (what an FC sees
 * while tokens are generated, and a short prefill chunk): the rows are fetched into device memory by a
 * small kernel, the product kernels write their outputs straight into host memory, and one wait ends
 * the call -- two launches and a wait instead of a copy in, the launches, one copy out per output and
 * the wait. Page-locked operands (the context's allocator) are used where they lie; pageable ones pass
 * through the stream's page-locked staging buffer with a memcpy on either side. Measured on page-locked
 * operands, us a call, copy engines -> this path: Q4_0 3072 x 1024 with 9 / 16 / 32 / 64 / 128 rows
 * 32 -> 19 / 34 -> 21 / 41 -> 28 / 52 -> 40 / 70 -> 60, Q4_K 4096 x 4096 42 -> 28 / 45 -> 32 / 56 -> 45 /
 * 78 -> 69 / 120 -> 115; at 256 rows the copy engines are level or ahead (111 against 105, 199 against 206). */
constexpr int64_t DIRECT_ROWS = 128;
constexpr size_t DIRECT_BYTES = (size_t)2 << 20; /* rows in, and all outputs together */
struct DirectIO {
  struct Out {
    float *host, *dev; /* where the caller wants it; where the kernels write (device-side address) */
    int64_t hld, dld, N;
    float *bounce; /* host address of the staging the kernels write, or null */
  };
  hipStream_t s = nullptr;
  int64_t rows = 0;
  const float *a_dev = nullptr; /* device-side address of the rows to fetch */
  int64_t a_ld = 0;
  std::vector<Out> outs;

  /* false: the call does not qualify (too many rows or bytes, odd K) and takes the copy engines */
  bool begin(hipStream_t stream, const float *A, int64_t M, int64_t lda, int64_t K, int count, float *const *C,
             const int64_t *ldc, const int64_t *Ns, int *rc) {
    *rc = HIPQ_OK;
    if (M < 1 || M > DIRECT_ROWS || (K & 3) || (size_t)M * K * 4 > DIRECT_BYTES) return false;
    size_t out_bytes = 0, stage_bytes = 0;
    for (int i = 0; i < count; ++i) out_bytes += (size_t)M * Ns[i] * 4;
    if (out_bytes > DIRECT_BYTES) return false;
    s = stream;
    rows = M;
    const bool a_direct = !(lda & 3) && !((uintptr_t)A & 15) && pinned_device_ptr(A);
    if (!a_direct) stage_bytes += ((size_t)M * K * 4 + 255) & ~(size_t)255;
    outs.resize(count);
    for (int i = 0; i < count; ++i) {
      outs[i] = Out{C[i], (float *)pinned_device_ptr(C[i]), ldc[i], ldc[i], Ns[i], nullptr};
      if (!outs[i].dev) stage_bytes += ((size_t)M * Ns[i] * 4 + 255) & ~(size_t)255;
    }
    char *stage = nullptr;
    if (stage_bytes) {
      void *p = nullptr;
      if ((*rc = pinned_staging(s, stage_bytes, &p))) return false;
      stage = (char *)p;
    }
    if (a_direct) {
      a_dev = (const float *)pinned_device_ptr(A);
      a_ld = lda;
    } else {
      for (int64_t r = 0; r < M; ++r) memcpy(stage + (size_t)r * K * 4, A + r * lda, (size_t)K * 4);
      a_dev = (const float *)pinned_device_ptr(stage);
      a_ld = K;
      stage += ((size_t)M * K * 4 + 255) & ~(size_t)255;
    }
    for (Out &o : outs)
      if (!o.dev) {
        o.bounce = (float *)stage;
        o.dev = (float *)pinned_device_ptr(stage);
        o.dld = o.N;
        stage += ((size_t)M * o.N * 4 + 255) & ~(size_t)255;
      }
    return true;
  }
  /* the rows into dense device memory dst [rows x K] */
  int fetch(float *dst, int64_t K) const {
    const int64_t quads = rows * K / 4;
    hipq::launch_kernel("fetch_rows_kernel", fetch_rows_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s, a_dev,
                        a_ld, dst, (int)K, (int)rows);
    HIPQ_HIP(hipGetLastError());
    return HIPQ_OK;
  }
  /* waits for the kernels; staged outputs go to where the caller wants them */
  int finish() const {
    if (int rc = wait_done(s)) return rc;
    for (const Out &o : outs)
      if (o.bounce)
        for (int64_t r = 0; r < rows; ++r) memcpy(o.host + r * o.hld, o.bounce + r * o.N, (size_t)o.N * 4);
    return HIPQ_OK;
  }
};

/* rows x width bytes between host (pitch hpitch) and a dense device buffer, in order on s.
 * to_device: the copy is queued when this returns (the host bytes have been read). Otherwise
 * the host bytes are written when this returns. */
int stage_copy(bool to_device, void *dev, void *host, size_t hpitch, size_t width, size_t rows, hipStream_t s) {
  if (!rows || !width) return HIPQ_OK;
  if (is_pinned(host)) {
    if (to_device) {
      HIPQ_HIP(hipMemcpy2DAsync(dev, width, host, hpitch, width, rows, hipMemcpyHostToDevice, s));
    } else {
      HIPQ_HIP(hipMemcpy2DAsync(host, hpitch, dev, width, width, rows, hipMemcpyDeviceToHost, s));
      HIPQ_HIP(hipStreamSynchronize(s));
    }
    return HIPQ_OK;
  }
  std::lock_guard<std::mutex> lk(g_ring.mu);
  int rc = g_ring.ensure();
  if (rc) return rc;
  constexpr int SLOTS = StageRing::SLOTS;
  /* a slice = as many whole rows as fit a slot, or a piece of one long row */
  const size_t rows_per = width <= StageRing::SLOT_BYTES ? StageRing::SLOT_BYTES / width : 0;
  struct Slice {
    size_t row, off, nrows, bytes; /* nrows rows from `row`, or `bytes` of row `row` from byte `off` */
  };
  auto slice_at = [&](size_t i, Slice &sl) -> bool {
    if (rows_per) {
      sl.row = i * rows_per;
      if (sl.row >= rows) return false;
      sl.off = 0;
      sl.nrows = rows - sl.row < rows_per ? rows - sl.row : rows_per;
      sl.bytes = sl.nrows * width;
      return true;
    }
    const size_t per_row = (width + StageRing::SLOT_BYTES - 1) / StageRing::SLOT_BYTES;
    sl.row = i / per_row;
    if (sl.row >= rows) return false;
    sl.off = (i % per_row) * StageRing::SLOT_BYTES;
    sl.nrows = 1;
    sl.bytes = width - sl.off < StageRing::SLOT_BYTES ? width - sl.off : StageRing::SLOT_BYTES;
    return true;
  };
  auto host_rows = [&](const Slice &sl, char *slot, bool into_slot) {
    if (hpitch == width || sl.nrows == 1) {
      char *h = (char *)host + sl.row * hpitch + sl.off;
      if (into_slot) memcpy(slot, h, sl.bytes); else memcpy(h, slot, sl.bytes);
      return;
    }
    for (size_t r = 0; r < sl.nrows; ++r) {
      char *h = (char *)host + (sl.row + r) * hpitch;
      if (into_slot) memcpy(slot + r * width, h, width); else memcpy(h, slot + r * width, width);
    }
  };
  Slice sl;
  const size_t p0 = g_ring.pos; /* slice i uses slot (p0 + i) % SLOTS */
  if (to_device) {
    size_t i = 0;
    for (; slice_at(i, sl); ++i) {
      const int k = (int)((p0 + i) % SLOTS);
      if ((rc = g_ring.wait_free(k))) return rc; /* also a slot an earlier transfer left in flight */
      host_rows(sl, g_ring.base + k * StageRing::SLOT_BYTES, true);
      HIPQ_HIP(hipMemcpyAsync((char *)dev + sl.row * width + sl.off, g_ring.base + k * StageRing::SLOT_BYTES, sl.bytes,
                              hipMemcpyHostToDevice, s));
      HIPQ_HIP(hipEventRecord(g_ring.ev[k], s));
      g_ring.busy[k] = true;
    }
    g_ring.pos = p0 + i;
    return HIPQ_OK;
  }
  size_t issued = 0, done = 0;
  for (;;) {
    while (issued < done + SLOTS && slice_at(issued, sl)) {
      const int k = (int)((p0 + issued) % SLOTS);
      if ((rc = g_ring.wait_free(k))) return rc;
      HIPQ_HIP(hipMemcpyAsync(g_ring.base + k * StageRing::SLOT_BYTES, (char *)dev + sl.row * width + sl.off, sl.bytes,
                              hipMemcpyDeviceToHost, s));
      HIPQ_HIP(hipEventRecord(g_ring.ev[k], s));
      g_ring.busy[k] = true;
      ++issued;
    }
    if (done == issued) break;
    const int k = (int)((p0 + done) % SLOTS);
    if ((rc = g_ring.wait_free(k))) return rc;
    slice_at(done, sl);
    host_rows(sl, g_ring.base + k * StageRing::SLOT_BYTES, false);
    ++done;
  }
  g_ring.pos = p0 + issued;
  return HIPQ_OK;
}

/* Rows of a host-memory call in steps. With page-locked operands the copies are asynchronous, and
 * the link carries both directions at once: while the kernels work on one step's rows, the copy
 * engines take the step before out (on a second stream) and, behind the kernels, bring the next
 * one in. A call of 512 rows and more is cut into steps of 256 (the last one takes the remainder)
 * where the caller says that every step's product has the bits of the whole call's, and where the
 * outputs are at least twice the input and 16 MiB: measured on page-locked memory (us, one piece -> steps),
 * 12288 x 4096 with 512 / 1024 / 2048 rows 675 -> 613 / 1315 -> 1102 / 2598 -> 2081, 4096 x 1024
 * 229 -> 225 / 428 -> 400 / 825 -> 754; with the input the larger side (1024 x 3072: 190 -> 214 /
 * 347 -> 395 / 661 -> 763) the steps' extra waits cost more than the little output they hide. */
struct RowSteps {
  static constexpr int64_t STEP = 256;
  static constexpr int64_t MIN_OUT_BYTES = (int64_t)16 << 20; /* below, a step's copy is too short to hide anything */
  hipStream_t s = nullptr, cs = nullptr;
  hipEvent_t ev = nullptr;
  int64_t M = 0, step = 0; /* step 0: the whole call in one piece */
  bool pending = false;

  int plan(hipStream_t stream, int64_t rows, bool steps_keep_bits, const float *A, int64_t in_cols, int count,
           float *const *C, int64_t out_cols) {
    s = stream;
    M = rows;
    step = 0;
    if (!steps_keep_bits || rows < 2 * STEP || out_cols < 2 * in_cols || rows * out_cols * 4 < MIN_OUT_BYTES ||
        !is_pinned(A))
      return HIPQ_OK;
    for (int i = 0; i < count; ++i)
      if (!is_pinned(C[i])) return HIPQ_OK;
    {
      std::lock_guard<std::mutex> lk(g.mu);
      Workspace &w = g.ws[s];
      if (!w.copy) HIPQ_HIP(hipStreamCreateWithFlags(&w.copy, hipStreamNonBlocking));
      if (!w.step_done) HIPQ_HIP(hipEventCreateWithFlags(&w.step_done, hipEventDisableTiming));
      cs = w.copy;
      ev = w.step_done;
    }
    step = STEP;
    return HIPQ_OK;
  }
  /* the rows of the piece that starts at r0 */
  int64_t rows_at(int64_t r0) const { return (!step || M - r0 < 2 * step) ? M - r0 : step; }
  int in(float *dev, const float *host, int64_t lda, int64_t K, int64_t r0, int64_t n) const {
    return stage_copy(true, dev + r0 * K, (void *)(host + r0 * lda), (size_t)lda * 4, (size_t)K * 4, (size_t)n, s);
  }
  /* rows [r0, r0 + n) of a dense device result [M x N] to the caller's matrix; in one piece this returns
   * with the host bytes written, in steps finish() does */
  int out(const float *dev, float *host, int64_t ldc, int64_t N, int64_t r0, int64_t n, bool first_of_step = true) {
    if (!step)
      return stage_copy(false, (void *)(dev + r0 * N), host + r0 * ldc, (size_t)ldc * 4, (size_t)N * 4, (size_t)n, s);
    if (first_of_step) {
      HIPQ_HIP(hipEventRecord(ev, s));
      HIPQ_HIP(hipStreamWaitEvent(cs, ev, 0));
    }
    pending = true;
    HIPQ_HIP(hipMemcpy2DAsync(host + r0 * ldc, (size_t)ldc * 4, dev + r0 * N, (size_t)N * 4, (size_t)N * 4, (size_t)n,
                              hipMemcpyDeviceToHost, cs));
    return HIPQ_OK;
  }
  int finish() {
    if (!pending) return HIPQ_OK;
    pending = false;
    HIPQ_HIP(hipStreamSynchronize(cs));
    return HIPQ_OK;
  }
  ~RowSteps() { /* a call that fails half way still owns the caller's memory until its copies end */
    if (pending) (void)hipStreamSynchronize(cs);
  }
};

std::recursive_mutex &enqueue_lock(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g.mu);
  return g.ws[s].enqueue; /* nodes of the map do not move */
}
typedef std::lock_guard<std::recursive_mutex> EnqueueGuard;

bool dtype_ok(int dt) { return dt == HIPQ_Q4_0 || dt == HIPQ_Q4_K || dt == HIPQ_Q6_K; }
int64_t block_elems(int dt) { return dt == HIPQ_Q4_0 ? 32 : 256; }
int64_t block_bytes(int dt) { return dt == HIPQ_Q4_0 ? 18 : dt == HIPQ_Q4_K ? 144 : 210; }

QAct qact_rows(const QAct &a, int is_k, int64_t r0, int64_t rows) {
  QAct v = a;
  v.q = a.q + r0 * a.K;
  if (is_k) {
    v.d = a.d + r0 * (a.K / 256);
    v.bsum = a.bsum + r0 * (a.K / 16);
    v.ql = a.ql + r0 * (a.K / 2);
    v.qh = a.qh + r0 * (a.K / 2);
  } else {
    v.meta = a.meta + r0 * (a.K / 32);
  }
  v.M = (int)rows;
  return v;
}

/* The prefill GEMMs of the K-formats take their activations in the tiled form. The Q4_K one
 * addresses the weight planes with 32-bit byte offsets where it has no tile copy; the Q6_K
 * one reads the tile copy only, which the entry point that may not allocate cannot build
 * (such a call then walks the rows eight at a time through the GEMV engine, as calls with few
 * rows do, and keeps the reference's bits). */
bool wants_tiled(const hipq_weight *w, int64_t M, bool may_allocate = true) {
  if (w->dtype == HIPQ_Q6_K) {
    /* The GEMV engine keeps the reference's bits but costs a pass over the weights per eight rows
     * and about 1e-7 us per weight and row on the vector ALU; the matrix-core GEMM costs one 64-row
     * tile whatever the row count (17-23 us in parts of K, or 2e-7 us per weight). Measured, us,
     * engine against GEMM: 151936 x 4096 with 2 / 4 / 8 / 16 rows 115 / 192 / 441 / 847 against 130;
     * 12288 x 4096 with 4 / 8 / 16 rows 22 / 42 / 80 against 23; 4096 x 4096 with 8 / 9 / 16 rows
     * 19 / 25 / 34 against 17. */
    const int64_t weights = w->N * w->K;
    const int64_t engine_rows = weights >= (int64_t(1) << 28) ? 2 : weights >= (int64_t(1) << 25) ? 4 :
                                weights >= (int64_t(1) << 24) ? 8 : 16;
    return M > engine_rows && (w->gt_base || may_allocate);
  }
  /* up to 16 rows of a Q4_K matrix of 1024 columns or more take the few-rows kernel (wants_rows) */
  if (hipq::gemm_rows_q4k_fits(w, M) && (w->gt_base || may_allocate)) return false;
  return w->dtype == HIPQ_Q4_K && M > 8 && w->N * (w->K / 2) < (int64_t(1) << 32);
}

/* Where a call's quantized activations go: the per-stream workspace (grown on
 * demand) or, for the entry point that may not allocate, the static scratch. */
struct Scratch {
  bool fixed;
  hipStream_t s;
  void *slot = nullptr; /* fixed: this stream's part of the static array */
  int get(size_t bytes, void **out) const {
    if (!fixed) return workspace(s, bytes, out);
    if (bytes > NOALLOC_SCRATCH_BYTES)
      return fail(HIPQ_ERR_NOT_SUPPORTED,
                  "this matmul needs %zu bytes of scratch for its quantized activations; the "
                  "allocation-free entry point holds %zu a stream",
                  bytes, NOALLOC_SCRATCH_BYTES);
    *out = slot;
    return HIPQ_OK;
  }
};

/* The slot of the static array that belongs to stream s (the first four streams that use the
 * allocation-free entry point get one each, until hipq_stream_release gives it back). */
int noalloc_slot(hipStream_t s, void **out) {
  std::lock_guard<std::mutex> lk(g.mu);
  int free_slot = -1;
  for (int i = 0; i < NOALLOC_SLOTS; ++i) {
    if (g.noalloc_taken[i] && g.noalloc_stream[i] == s) {
      *out = (char *)g.scratch_ptr[g.device] + (size_t)i * NOALLOC_SCRATCH_BYTES;
      return HIPQ_OK;
    }
    if (!g.noalloc_taken[i] && free_slot < 0) free_slot = i;
  }
  if (free_slot < 0)
    return fail(HIPQ_ERR_NOT_SUPPORTED,
                "%d streams already use the allocation-free entry point, one slot of its scratch each; "
                "hipq_stream_release gives a stream's slot back",
                NOALLOC_SLOTS);
  g.noalloc_taken[free_slot] = true;
  g.noalloc_stream[free_slot] = s;
  *out = (char *)g.scratch_ptr[g.device] + (size_t)free_slot * NOALLOC_SCRATCH_BYTES;
  return HIPQ_OK;
}

int matmul_tiled(const hipq_weight *w, const float *A, int64_t M, int64_t lda, float *C, int64_t ldc,
                 hipStream_t s, int phase, const Scratch &sc);

/* Quantize the activations the way the reference does for this weight type. */
int quantize_for(const hipq_weight *w, const float *A, int64_t M, int64_t lda, const QAct &qa,
                 hipStream_t s, bool each_row = false) {
  if (w->dtype == HIPQ_Q4_0) return hipq::launch_quantize_q8_0(A, M, w->K, lda, &qa, nullptr, s);
  const int64_t mat_rows = (w->dtype == HIPQ_Q4_K && M > 1 && !each_row) ? (M / 4) * 4 : 0;
  return hipq::launch_quantize_q8_K(A, M, w->K, lda, mat_rows, &qa, nullptr, s);
}

/* Block-dot stage on already quantized activations. */
int multiply(const hipq_weight *w, const QAct &qa, int64_t M, float *C, int64_t ldc,
             hipStream_t s, bool each_row = false) {
  const int is_k = w->dtype != HIPQ_Q4_0;
  /* rows the reference sends through its 4-row GEMM kernel (Q4_K, M > 1) */
  const int pair_rows = (w->dtype == HIPQ_Q4_K && M > 1 && !each_row) ? (int)((M / 4) * 4) : 0;
  /* Q4_0: every kernel carries the reference's bits, so the row count only picks the fastest. A few
   * rows (up to 64 where the launch stays small) go to the few-rows kernel of gemm_rows_q40.hip; where
   * that one does not apply (narrow matrices), the prefill GEMM also takes five to eight rows from
   * 2^25 weights up, where the GEMV engine's eight-row pass is the slower of the two */
  const bool q40_gemm = w->dtype == HIPQ_Q4_0 && w->K % 256 == 0;
  if (hipq::gemm_rows_q40_fits(w, M)) return hipq::launch_gemm_rows_q40(w, &qa, (int)M, C, ldc, s);
  if (M <= 8 && !(q40_gemm && M >= 5 && w->N * w->K >= (int64_t(1) << 25)))
    return hipq::launch_gemv(w, &qa, (int)M, pair_rows, C, ldc, s);
  if (q40_gemm) return hipq::launch_gemm(w, &qa, (int)M, C, ldc, s);
  for (int64_t r0 = 0; r0 < M; r0 += 8) {
    const int64_t rows = (M - r0) < 8 ? (M - r0) : 8;
    QAct sub = qact_rows(qa, is_k, r0, rows);
    int rc = hipq::launch_gemv(w, &sub, (int)rows, 0, C + r0 * ldc, ldc, s);
    if (rc) return rc;
  }
  return HIPQ_OK;
}

int check_matmul_args(hipq_weight_t w, const float *A, int64_t M, int64_t lda, const float *C,
                      int64_t ldc) {
  if (!w || !A || !C) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null weight, activation or output");
  if (w->expert_tiles)
    return fail(HIPQ_ERR_INVALID_ARGUMENT,
                "the weight has been an expert of hipq_moe_forward and is stored for that use only");
  if (M < 0) return fail(HIPQ_ERR_INVALID_ARGUMENT, "M = %lld", (long long)M);
  if (lda < w->K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "lda %lld < K %lld", (long long)lda, (long long)w->K);
  if (ldc < w->N) return fail(HIPQ_ERR_INVALID_ARGUMENT, "ldc %lld < N %lld", (long long)ldc, (long long)w->N);
  return HIPQ_OK;
}

/* phase: 0 quantizer + GEMM, 1 GEMM only (activations from the previous call), 2 quantizer only */
int matmul_tiled(const hipq_weight *w, const float *A, int64_t M, int64_t lda, float *C, int64_t ldc,
                 hipStream_t s, int phase, const Scratch &sc) {
  void *mem = nullptr;
  /* The GEMM reads a tile copy of the weights (coalesced loads), made at the weight's first
   * prefill product (before anything that depends on its existence, so that the first product has
   * the bits of the following ones); the entry point that may not allocate reads the planes
   * until it exists. */
  if (!w->gt_base && !sc.fixed) {
    const int trc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(w));
    if (trc) return trc;
  }
  /* room for the partial products of a product with few tiles behind the activations (the fixed
   * scratch of the allocation-free entry point may be too small for them: then none) */
  const size_t act_bytes = (qact_tiled_bytes(M, w->K) + 255) & ~(size_t)255;
  size_t part_bytes = w->dtype == HIPQ_Q4_K ? hipq::gemm_q4k_split_bytes(w, M) : hipq::gemm_q6k_split_bytes(w, M);
  if (sc.fixed && act_bytes + part_bytes > NOALLOC_SCRATCH_BYTES) part_bytes = 0;
  int rc = sc.get(act_bytes + part_bytes, &mem);
  if (rc) return rc;
  QActTiled qa = qact_tiled_carve(mem, M, w->K);
  void *partials = part_bytes ? (char *)mem + act_bytes : nullptr;
  /* rows below the last multiple of four follow the 4-row quantizer for Q4_K (what the
   * reference's GEMM wrapper calls for them); its Q6_K path quantizes row by row */
  const int64_t mat_rows = w->dtype == HIPQ_Q4_K ? (M / 4) * 4 : 0;
  if (phase != 1) rc = hipq::launch_quantize_q8_K_tiled(A, M, w->K, lda, mat_rows, &qa, s);
  if (rc || phase == 2) return rc;
  if (w->dtype == HIPQ_Q6_K) return hipq::launch_gemm_q6k(w, &qa, (int)M, C, ldc, s, partials);
  return hipq::launch_gemm_q4k(w, &qa, (int)M, C, ldc, s, partials);
}

/* Three to eight rows of a large Q4_K matrix run on the matrix cores (gemm_rows_q4k.hip, the
 * reference's bits as the GEMV engine's) off the weight's tile copy; the entry point that may not
 * allocate takes that path only once the copy exists.
 * phase: 0 quantizer + product, 1 product only, 2 quantizer only */
bool wants_rows(const hipq_weight *w, int64_t M, bool may_allocate) {
  return hipq::gemm_rows_q4k_fits(w, M) && (w->gt_base || may_allocate);
}

int matmul_rows(const hipq_weight *w, const float *A, int64_t M, int64_t lda, float *C, int64_t ldc,
                hipStream_t s, int phase, const Scratch &sc, bool each_row = false) {
  void *mem = nullptr;
  int rc = sc.get(qact_bytes(1, M, w->K), &mem);
  if (rc) return rc;
  QAct qa = qact_carve(1, mem, M, w->K);
  const int64_t mat_rows = each_row ? 0 : (M / 4) * 4; /* the rows the reference quantizes four at a time */
  if (phase != 1) rc = hipq::launch_quantize_q8_K_rowmma(A, M, w->K, lda, &qa, s, mat_rows);
  if (rc || phase == 2) return rc;
  if (!w->gt_base && (rc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(w)))) return rc;
  return hipq::launch_gemm_rows_q4k(w, &qa, (int)M, (int)mat_rows, C, ldc, s); /* up to two passes of eight rows */
}

/* each_row: every row as a product of its own with M = 1 (the bits of M separate calls): for Q4_0
 * and Q6_K that is what up to 16 rows give anyway; Q4_K drops the 4-row quantizer and the pairwise
 * sums the reference applies to rows it multiplies together. The caller passes at most 16 rows. */
int matmul_device(hipq_weight_t w, const float *A, int64_t M, int64_t lda, float *C, int64_t ldc,
                  hipStream_t s, const Scratch &sc, bool each_row = false) {
  if (M == 0) return HIPQ_OK;
  if (wants_rows(w, M, !sc.fixed)) return matmul_rows(w, A, M, lda, C, ldc, s, 0, sc, each_row);
  if (!each_row && wants_tiled(w, M, !sc.fixed)) return matmul_tiled(w, A, M, lda, C, ldc, s, 0, sc);
  if (M == 1 && hipq::gemv_fuses_quantizer(w, A)) return hipq::launch_gemv_fused(w, A, C, s);
  {
    const hipq_weight *one = w;
    if (hipq::gemm_rows_q40_fuses(1, &one, M, A, lda)) return hipq::launch_gemm_rows_q40_fused(1, &one, A, lda, (int)M, &C, &ldc, s);
  }
  const int is_k = w->dtype != HIPQ_Q4_0;
  void *mem = nullptr;
  int rc = sc.get(qact_bytes(is_k, M, w->K), &mem);
  if (rc) return rc;
  QAct qa = qact_carve(is_k, mem, M, w->K);
  rc = quantize_for(w, A, M, lda, qa, s, each_row);
  if (rc) return rc;
  if (each_row && w->dtype == HIPQ_Q4_K && M > 8) { /* nine to sixteen rows of a small matrix: two GEMV passes */
    for (int64_t r0 = 0; r0 < M && !rc; r0 += 8) {
      const int64_t rows = (M - r0) < 8 ? (M - r0) : 8;
      const QAct sub = qact_rows(qa, 1, r0, rows);
      rc = hipq::launch_gemv(w, &sub, (int)rows, 0, C + r0 * ldc, ldc, s);
    }
    return rc;
  }
  return multiply(w, qa, M, C, ldc, s, each_row);
}

/* Whether the products of a call of M rows against these weights have the same bits when the rows are
 * multiplied in steps of RowSteps::STEP (the last one up to twice that). Q4_0: every kernel has the
 * reference's bits, always. Q4_K and Q6_K: where the whole call and every step take the prefill GEMM
 * on whole K (a row's sums there depend on neither the other rows nor the tile height; a product in
 * parts of K adds in another order). The weights' tile copies are made here, as the products would. */
int steps_keep_bits(int count, const hipq_weight_t *w, int64_t M, bool *keep) {
  *keep = false;
  if (M < 2 * RowSteps::STEP) return HIPQ_OK;
  const int64_t sizes[3] = {M, RowSteps::STEP, RowSteps::STEP + M % RowSteps::STEP};
  for (int i = 0; i < count; ++i) {
    if (w[i]->dtype == HIPQ_Q4_0) continue;
    for (int64_t m : sizes)
      if (!wants_tiled(w[i], m)) return HIPQ_OK;
    if (!w[i]->gt_base)
      if (int rc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(w[i]))) return rc;
    for (int64_t m : sizes)
      if (w[i]->dtype == HIPQ_Q4_K ? hipq::gemm_q4k_split_bytes(w[i], m) : hipq::gemm_q6k_split_bytes(w[i], m))
        return HIPQ_OK;
  }
  *keep = true;
  return HIPQ_OK;
}

struct DevBuf {
  void *p = nullptr;
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
  int alloc(size_t n) {
    hipError_t e = hipMalloc(&p, n ? n : 16);
    if (e != hipSuccess) {
      p = nullptr;
      return fail(HIPQ_ERR_OUT_OF_MEMORY, "hipMalloc(%zu): %s", n, hipGetErrorString(e));
    }
    return HIPQ_OK;
  }
};

} // namespace

extern "C" {

const char *hipq_last_error(void) { return tl_error; }
const char *hipq_version(void) { return "0.1"; }

int hipq_init(int device) {
  std::lock_guard<std::mutex> lk(g.mu);
  if (g.ready) {
    if (g.device == device) return HIPQ_OK;
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "already initialised on device %d", g.device);
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return fail(HIPQ_ERR_RUNTIME, "no HIP device available (%s)", hipGetErrorString(e));
  if (device < 0 || device >= count)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "device %d out of range [0, %d)", device, count);
  hipDeviceProp_t prop;
  HIPQ_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(HIPQ_ERR_NOT_SUPPORTED, "device %d is %s; this library is built for gfx950 only",
                device, prop.gcnArchName);
  HIPQ_HIP(hipSetDevice(device));
  if (device >= MAX_DEVICES) return fail(HIPQ_ERR_NOT_SUPPORTED, "device index %d is beyond %d", device, MAX_DEVICES - 1);
  if (!g.scratch_ptr[device]) {
    void *p = nullptr;
    HIPQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g.scratch_ptr[device] = p;
  }
  g.device = device;
  g.ready = true;
  return HIPQ_OK;
}

int hipq_shutdown(void) {
  std::lock_guard<std::mutex> lk(g.mu);
  if (!g.ready) return HIPQ_OK;
  if (g.live_weights)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "%lld weights still alive", (long long)g.live_weights);
  (void)hipSetDevice(g.device);
  (void)hipDeviceSynchronize();
  for (auto &kv : g.ws) {
    if (kv.second.ptr) (void)hipFree(kv.second.ptr);
    if (kv.second.io) (void)hipFree(kv.second.io);
    if (kv.second.pin) (void)hipHostFree(kv.second.pin);
    if (kv.second.done) (void)hipHostFree(kv.second.done);
    if (kv.second.step_done) (void)hipEventDestroy(kv.second.step_done);
    if (kv.second.copy) (void)hipStreamDestroy(kv.second.copy);
    for (void *p : kv.second.retired) (void)hipFree(p);
  }
  g.ws.clear();
  for (int i = 0; i < NOALLOC_SLOTS; ++i) g.noalloc_taken[i] = false;
  {
    std::lock_guard<std::mutex> rl(g_ring.mu);
    if (g_ring.base) {
      for (int i = 0; i < StageRing::SLOTS; ++i) (void)hipEventDestroy(g_ring.ev[i]);
      (void)hipHostFree(g_ring.base);
      g_ring.base = nullptr;
    }
  }
  for (auto &kv : g.moe_tables)
    if (kv.second.dev) (void)hipFree(kv.second.dev);
  g.moe_tables.clear();
  g.ready = false;
  g.device = -1;
  return HIPQ_OK;
}

int hipq_stream_release(void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  std::lock_guard<std::mutex> lk(g.mu);
  for (int i = 0; i < NOALLOC_SLOTS; ++i) /* its slot of the allocation-free scratch, if it has one */
    if (g.noalloc_taken[i] && g.noalloc_stream[i] == s) {
      HIPQ_HIP(hipStreamSynchronize(s));
      g.noalloc_taken[i] = false;
    }
  auto it = g.ws.find(s);
  if (it == g.ws.end()) return HIPQ_OK;
  /* a caller that still enqueues on the stream from another thread holds the lock: refuse */
  std::unique_lock<std::recursive_mutex> el(it->second.enqueue, std::try_to_lock);
  if (!el.owns_lock() || it->second.depth)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the stream is in use by another call");
  HIPQ_HIP(hipStreamSynchronize(s));
  if (it->second.ptr) (void)hipFree(it->second.ptr);
  if (it->second.io) (void)hipFree(it->second.io);
  if (it->second.pin) (void)hipHostFree(it->second.pin);
  if (it->second.done) (void)hipHostFree(it->second.done);
  if (it->second.step_done) (void)hipEventDestroy(it->second.step_done);
  if (it->second.copy) (void)hipStreamDestroy(it->second.copy);
  for (void *p : it->second.retired) (void)hipFree(p);
  el.unlock();
  el.release();
  g.ws.erase(it);
  return HIPQ_OK;
}

int hipq_host_alloc(void **ptr, size_t bytes) {
  int rc = require_ready();
  if (rc) return rc;
  if (!ptr) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  *ptr = nullptr;
  hipError_t e = hipHostMalloc(ptr, bytes ? bytes : 16, hipHostMallocDefault);
  if (e != hipSuccess) {
    *ptr = nullptr;
    return fail(HIPQ_ERR_OUT_OF_MEMORY, "hipHostMalloc(%zu): %s", bytes, hipGetErrorString(e));
  }
  memset(*ptr, 0, bytes); /* as the framework's default allocator (calloc, mem_allocator.cpp:22-27) */
  return HIPQ_OK;
}

int hipq_host_free(void *ptr) {
  if (!ptr) return HIPQ_OK;
  int rc = require_ready();
  if (rc) return rc;
  HIPQ_HIP(hipHostFree(ptr));
  return HIPQ_OK;
}

int64_t hipq_weight_nbytes(int dtype, int64_t N, int64_t K) {
  if (!dtype_ok(dtype)) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown weight dtype %d", dtype);
  if (N <= 0 || K <= 0 || K % block_elems(dtype))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "N=%lld K=%lld: K must be a positive multiple of %lld",
                (long long)N, (long long)K, (long long)block_elems(dtype));
  return N * (K / block_elems(dtype)) * block_bytes(dtype);
}

int hipq_weight_create(int dtype, int layout, int64_t N, int64_t K, const void *bytes, int mem,
                       hipq_weight_t *out) {
  int rc = require_ready();
  if (rc) return rc;
  if (!out || !bytes) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  *out = nullptr;
  const int64_t nbytes = hipq_weight_nbytes(dtype, N, K);
  if (nbytes < 0) return (int)nbytes;
  if (layout != HIPQ_LAYOUT_CANONICAL && layout != HIPQ_LAYOUT_X8)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown layout %d", layout);
  if (layout == HIPQ_LAYOUT_X8) {
    if (dtype == HIPQ_Q6_K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "Q6_K has no x8 layout");
    /* same rule as the reference's repack: 8 rows interleaved, K % 8 == 0 */
    if (N % 8 || K % 8)
      return fail(HIPQ_ERR_INVALID_ARGUMENT, "x8 layout needs N %% 8 == 0 and K %% 8 == 0 (N=%lld K=%lld)",
                  (long long)N, (long long)K);
  }
  if (N > INT32_MAX || K > INT32_MAX) return fail(HIPQ_ERR_INVALID_ARGUMENT, "dimension too large");

  hipq_weight *w = new (std::nothrow) hipq_weight();
  if (!w) return fail(HIPQ_ERR_OUT_OF_MEMORY, "host allocation failed");
  w->dtype = dtype;
  w->device = g.device;
  w->expert_tiles = 0;
  w->gt_base = nullptr;
  w->gt_qs = w->gt_qh = w->gt_hdr = nullptr;
  w->N = N;
  w->K = K;
  /* planes, each 256-byte aligned */
  auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  size_t o_qs = 0, o_qh = 0, o_hdr = 0, o_sc = 0, o_d = 0, total = 0;
  if (dtype == HIPQ_Q4_0) {
    o_qs = 0;
    o_d = up((size_t)N * K / 2);
    total = o_d + up((size_t)N * (K / 32) * 2);
  } else if (dtype == HIPQ_Q4_K) {
    o_qs = 0;
    o_hdr = up((size_t)N * K / 2);
    total = o_hdr + up((size_t)N * (K / 256) * 16);
  } else {
    o_qs = 0;
    o_qh = up((size_t)N * K / 2);
    o_sc = o_qh + up((size_t)N * K / 4);
    o_d = o_sc + up((size_t)N * K / 16);
    total = o_d + up((size_t)N * (K / 256) * 2);
  }
  hipError_t e = hipMalloc((void **)&w->base, total);
  if (e != hipSuccess) {
    delete w;
    return fail(HIPQ_ERR_OUT_OF_MEMORY, "weight planes of %zu bytes: %s", total, hipGetErrorString(e));
  }
  w->bytes = total;
  w->qs = w->base + o_qs;
  w->qh = dtype == HIPQ_Q6_K ? w->base + o_qh : nullptr;
  w->hdr = dtype == HIPQ_Q4_K ? w->base + o_hdr : nullptr;
  w->sc = dtype == HIPQ_Q6_K ? (const int8_t *)(w->base + o_sc) : nullptr;
  w->d = dtype != HIPQ_Q4_K ? (const uint16_t *)(w->base + o_d) : nullptr;

  const uint8_t *src = (const uint8_t *)bytes;
  DevBuf staging;
  if (mem == HIPQ_MEM_HOST) {
    rc = staging.alloc((size_t)nbytes);
    if (!rc) {
      e = hipMemcpy(staging.p, bytes, (size_t)nbytes, hipMemcpyHostToDevice);
      if (e != hipSuccess) rc = fail(HIPQ_ERR_RUNTIME, "weight upload: %s", hipGetErrorString(e));
    }
    src = (const uint8_t *)staging.p;
  } else if (mem != HIPQ_MEM_DEVICE) {
    rc = fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  }
  if (!rc) rc = hipq::launch_relayout(w, layout, src, nullptr);
  if (!rc) {
    e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) rc = fail(HIPQ_ERR_RUNTIME, "weight relayout: %s", hipGetErrorString(e));
  }
  if (rc) {
    (void)hipFree(w->base);
    delete w;
    return rc;
  }
  {
    std::lock_guard<std::mutex> lk(g.mu);
    g.live_weights++;
  }
  *out = w;
  return HIPQ_OK;
}

int hipq_file_layout(int count, const hipq_file_tensor *tensors, int64_t offset, int64_t *data_offsets,
                     int64_t *end_offset) {
  if (count < 0 || (count && !tensors) || offset < 0)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad tensor list");
  int64_t at = offset;
  for (int i = 0; i < count; ++i) {
    const hipq_file_tensor &t = tensors[i];
    int64_t size;
    if (t.dtype == HIPQ_FILE_SKIP) {
      if (t.bytes < 0) return fail(HIPQ_ERR_INVALID_ARGUMENT, "tensor %d: negative size", i);
      size = t.bytes;
    } else {
      size = hipq_weight_nbytes(t.dtype, t.N, t.K);
      if (size < 0) return (int)size;
      if (t.dtype == HIPQ_Q4_K) at += 2; /* the scheme word comes first */
    }
    if (data_offsets) data_offsets[i] = at;
    at += size;
  }
  if (end_offset) *end_offset = at;
  return HIPQ_OK;
}

int hipq_weights_from_file(const char *path, int64_t offset, int count, const hipq_file_tensor *tensors,
                           hipq_weight_t *out, int64_t *end_offset) {
  int rc = require_ready();
  if (rc) return rc;
  if (!path || !out) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  std::vector<int64_t> at((size_t)(count > 0 ? count : 0));
  int64_t end = 0;
  if ((rc = hipq_file_layout(count, tensors, offset, at.data(), &end))) return rc;
  for (int i = 0; i < count; ++i) out[i] = nullptr;
  FILE *f = fopen(path, "rb");
  if (!f) return fail(HIPQ_ERR_INVALID_ARGUMENT, "cannot open %s", path);
  std::vector<unsigned char> buf;
  for (int i = 0; i < count && !rc; ++i) {
    const hipq_file_tensor &t = tensors[i];
    if (t.dtype == HIPQ_FILE_SKIP) continue;
    const int64_t size = hipq_weight_nbytes(t.dtype, t.N, t.K);
    if (t.dtype == HIPQ_Q4_K) {
      uint16_t scheme = 0;
      if (fseeko(f, (off_t)(at[i] - 2), SEEK_SET) || fread(&scheme, 2, 1, f) != 1)
        rc = fail(HIPQ_ERR_INVALID_ARGUMENT, "%s ends before tensor %d", path, i);
      else if (scheme == 0x03 && t.layout != HIPQ_LAYOUT_X8)
        rc = fail(HIPQ_ERR_INVALID_ARGUMENT, "tensor %d is stored as Q4_Kx8 but listed as canonical", i);
      if (rc) break;
    }
    buf.resize((size_t)size);
    if (fseeko(f, (off_t)at[i], SEEK_SET) || fread(buf.data(), 1, (size_t)size, f) != (size_t)size) {
      rc = fail(HIPQ_ERR_INVALID_ARGUMENT, "%s ends before the end of tensor %d", path, i);
      break;
    }
    rc = hipq_weight_create(t.dtype, t.layout, t.N, t.K, buf.data(), HIPQ_MEM_HOST, &out[i]);
  }
  fclose(f);
  if (rc) {
    for (int i = 0; i < count; ++i) {
      if (out[i]) (void)hipq_weight_destroy(out[i]);
      out[i] = nullptr;
    }
    return rc;
  }
  if (end_offset) *end_offset = end;
  return HIPQ_OK;
}

int hipq_weight_destroy(hipq_weight_t w) {
  if (!w) return HIPQ_OK;
  int rc = require_ready();
  if (rc) return rc;
  {
    /* no MoE call is between its table look-up and its launches while moe_mu is held, so
     * after the synchronization nothing on the device reads w or a table that names it */
    std::lock_guard<std::mutex> ml(g.moe_mu);
    (void)hipDeviceSynchronize();
    (void)hipFree(w->base);
    if (w->gt_base) (void)hipFree(w->gt_base);
    std::lock_guard<std::mutex> lk(g.mu);
    g.live_weights--;
    /* drop the expert tables that name w, and only those: the tables of other layers stay
     * valid, also for graphs captured with them */
    for (auto it = g.moe_tables.begin(); it != g.moe_tables.end();) {
      bool names = false;
      for (const hipq_weight *k : it->second.key) names = names || k == w;
      if (names) {
        if (it->second.dev) (void)hipFree(it->second.dev);
        it = g.moe_tables.erase(it);
      } else
        ++it;
    }
  }
  delete w;
  return HIPQ_OK;
}

int hipq_weight_dims(hipq_weight_t w, int *dtype, int64_t *N, int64_t *K) {
  if (!w) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null weight");
  if (dtype) *dtype = w->dtype;
  if (N) *N = w->N;
  if (K) *K = w->K;
  return HIPQ_OK;
}

/* ---- activation quantizers (canonical output) ---------------------------- */

static int quantize_api(int is_k, const float *A, int64_t M, int64_t K, int64_t lda, int variant,
                        void *out, int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!A || !out) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  if (M < 0 || K <= 0 || K % (is_k ? 256 : 32) || lda < K)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "M=%lld K=%lld lda=%lld", (long long)M, (long long)K, (long long)lda);
  if (is_k && variant != HIPQ_Q8K_ROW && variant != HIPQ_Q8K_MAT)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown Q8_K variant %d", variant);
  if (M == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t out_bytes = (size_t)M * (K / (is_k ? 256 : 32)) * (is_k ? 292 : 34);
  const int64_t mat_rows = (is_k && variant == HIPQ_Q8K_MAT) ? M : 0;
  if (mem == HIPQ_MEM_DEVICE) {
    return is_k ? hipq::launch_quantize_q8_K(A, M, K, lda, mat_rows, nullptr, out, s)
                : hipq::launch_quantize_q8_0(A, M, K, lda, nullptr, out, s);
  }
  if (mem != HIPQ_MEM_HOST) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  DevBuf dA, dOut;
  if ((rc = dA.alloc((size_t)M * K * 4))) return rc;
  if ((rc = dOut.alloc(out_bytes))) return rc;
  HIPQ_HIP(hipMemcpy2D(dA.p, (size_t)K * 4, A, (size_t)lda * 4, (size_t)K * 4, (size_t)M,
                       hipMemcpyHostToDevice));
  rc = is_k ? hipq::launch_quantize_q8_K((const float *)dA.p, M, K, K, mat_rows, nullptr, dOut.p, s)
            : hipq::launch_quantize_q8_0((const float *)dA.p, M, K, K, nullptr, dOut.p, s);
  if (rc) return rc;
  HIPQ_HIP(hipStreamSynchronize(s));
  HIPQ_HIP(hipMemcpy(out, dOut.p, out_bytes, hipMemcpyDeviceToHost));
  return HIPQ_OK;
}

int hipq_quantize_q8_0(const float *A, int64_t M, int64_t K, int64_t lda, void *out_blocks,
                       int mem, void *stream) {
  return quantize_api(0, A, M, K, lda, 0, out_blocks, mem, stream);
}

int hipq_quantize_q8_K(const float *A, int64_t M, int64_t K, int64_t lda, int variant,
                       void *out_blocks, int mem, void *stream) {
  return quantize_api(1, A, M, K, lda, variant, out_blocks, mem, stream);
}

/* ---- matmul --------------------------------------------------------------- */

int hipq_matmul(hipq_weight_t w, const float *A, int64_t M, int64_t lda, float *C, int64_t ldc,
                int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if ((rc = check_matmul_args(w, A, M, lda, C, ldc))) return rc;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);
  const Scratch sc{false, s};
  if (mem == HIPQ_MEM_DEVICE) return matmul_device(w, A, M, lda, C, ldc, s, sc);
  if (mem != HIPQ_MEM_HOST) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  if (M == 0) return HIPQ_OK;
  /* host operands: device copies in the stream's operand buffer (grown on demand, no
   * allocation per call), moved through the pinned ring */
  const size_t a_bytes = ((size_t)M * w->K * 4 + 255) & ~(size_t)255, c_bytes = (size_t)M * w->N * 4;
  void *io = nullptr;
  if ((rc = io_buffer(s, a_bytes + c_bytes, &io))) return rc;
  float *dA = (float *)io, *dC = (float *)((char *)io + a_bytes);
  {
    DirectIO dio; /* a decode step's rows: no copy engine */
    if (dio.begin(s, A, M, lda, w->K, 1, &C, &ldc, &w->N, &rc)) {
      if ((rc = dio.fetch(dA, w->K))) return rc;
      if ((rc = matmul_device(w, dA, M, w->K, dio.outs[0].dev, dio.outs[0].dld, s, sc))) return rc;
      return dio.finish();
    }
    if (rc) return rc;
  }
  bool keep = false;
  if ((rc = steps_keep_bits(1, &w, M, &keep))) return rc;
  RowSteps steps;
  if ((rc = steps.plan(s, M, keep, A, w->K, 1, &C, w->N))) return rc;
  for (int64_t r0 = 0; r0 < M;) {
    const int64_t n = steps.rows_at(r0);
    if ((rc = steps.in(dA, A, lda, w->K, r0, n))) return rc;
    if ((rc = matmul_device(w, dA + r0 * w->K, n, w->K, dC + r0 * w->N, w->N, s, sc))) return rc;
    if ((rc = steps.out(dC, C, ldc, w->N, r0, n))) return rc;
    r0 += n;
  }
  return steps.finish();
}

int hipq_matmul_each_row(hipq_weight_t w, const float *A, int64_t rows, int64_t lda, float *C, int64_t ldc,
                         int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if ((rc = check_matmul_args(w, A, rows, lda, C, ldc))) return rc;
  if (mem != HIPQ_MEM_DEVICE && mem != HIPQ_MEM_HOST) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  if (rows == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);
  const Scratch sc{false, s};
  const float *dA = A;
  float *dC = C;
  int64_t a_ld = lda, c_ld = ldc;
  bool direct = false;
  DirectIO dio;
  if (mem == HIPQ_MEM_HOST) {
    const size_t a_bytes = ((size_t)rows * w->K * 4 + 255) & ~(size_t)255, c_bytes = (size_t)rows * w->N * 4;
    void *io = nullptr;
    if ((rc = io_buffer(s, a_bytes + c_bytes, &io))) return rc;
    dA = (const float *)io, dC = (float *)((char *)io + a_bytes), a_ld = w->K, c_ld = w->N;
    if (dio.begin(s, A, rows, lda, w->K, 1, &C, &ldc, &w->N, &rc)) { /* a decode step's rows: no copy engine */
      if ((rc = dio.fetch((float *)io, w->K))) return rc;
      dC = dio.outs[0].dev, c_ld = dio.outs[0].dld;
      direct = true;
    } else if (rc || (rc = stage_copy(true, (void *)dA, (void *)A, (size_t)lda * 4, (size_t)w->K * 4, (size_t)rows, s)))
      return rc;
  }
  for (int64_t r0 = 0; r0 < rows && !rc;) { /* steps of row counts that keep the M = 1 bits */
    int64_t n = (rows - r0) < 16 ? (rows - r0) : 16;
    if (w->dtype == HIPQ_Q4_0) n = rows - r0; /* every product of this format has them */
    if (w->dtype == HIPQ_Q4_K) /* up to 64 where the few-rows kernel takes that many in one launch */
      for (int64_t c = 64; c > 16; c -= 8) {
        const int64_t t = (rows - r0) < c ? (rows - r0) : c;
        if (t > 16 && wants_rows(w, t, true)) {
          n = t;
          break;
        }
      }
    rc = matmul_device(w, dA + r0 * a_ld, n, a_ld, dC + r0 * c_ld, c_ld, s, sc, true);
    r0 += n;
  }
  if (rc || mem == HIPQ_MEM_DEVICE) return rc;
  if (direct) return dio.finish();
  return stage_copy(false, dC, C, (size_t)ldc * 4, (size_t)w->N * 4, (size_t)rows, s);
}

int hipq_matmul_noalloc(hipq_weight_t w, const float *A, int64_t M, int64_t lda, float *C,
                        int64_t ldc, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if ((rc = check_matmul_args(w, A, M, lda, C, ldc))) return rc;
  hipStream_t s = (hipStream_t)stream;
  /* calls submit one at a time; each stream has its own slot of the scratch, so the kernels of
   * calls on different streams do not share memory (two calls on ONE stream run in order) */
  EnqueueGuard eg(g.noalloc_enqueue);
  void *slot = nullptr;
  if ((rc = noalloc_slot(s, &slot))) return rc;
  return matmul_device(w, A, M, lda, C, ldc, s, Scratch{true, s, slot});
}

int hipq_mlp_swiglu(hipq_weight_t w_act, hipq_weight_t w_mul, const float *A, int64_t M, int64_t lda,
                    float *out, int64_t ldo, int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if ((rc = check_matmul_args(w_act, A, M, lda, out, ldo))) return rc;
  if ((rc = check_matmul_args(w_mul, A, M, lda, out, ldo))) return rc;
  if (w_act->K != w_mul->K || w_act->N != w_mul->N)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the two projections differ in shape");
  if (mem != HIPQ_MEM_DEVICE && mem != HIPQ_MEM_HOST)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  if (M == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);
  const int64_t N = w_act->N, K = w_act->K;
  const size_t a_bytes = ((size_t)M * K * 4 + 255) & ~(size_t)255, o_bytes = ((size_t)M * N * 4 + 255) & ~(size_t)255;
  if (mem == HIPQ_MEM_DEVICE && M == 1 && hipq::gemv_fuses_swiglu(w_act, w_mul, A))
    return hipq::launch_gemv_fused_swiglu(w_act, w_mul, A, out, s);
  /* otherwise: both products from one quantization into the stream's operand buffer, then the
   * activation; host operands cross through the same buffer */
  void *io = nullptr;
  if ((rc = io_buffer(s, a_bytes + 3 * o_bytes, &io))) return rc;
  float *dA = (float *)io, *dY = (float *)((char *)io + a_bytes), *dZ = (float *)((char *)dY + o_bytes),
        *dO = (float *)((char *)dZ + o_bytes);
  const float *a_dev = A;
  int64_t a_ld = lda;
  float *h_out = nullptr; /* a decode step's output: the device-side address the kernels write */
  int64_t h_ld = 0;
  DirectIO dio;
  if (mem == HIPQ_MEM_HOST) {
    if (dio.begin(s, A, M, lda, K, 1, &out, &ldo, &N, &rc)) {
      if ((rc = dio.fetch(dA, K))) return rc;
      h_out = dio.outs[0].dev, h_ld = dio.outs[0].dld;
    } else if (rc || (M == 1 && (rc = stage_copy(true, dA, (void *)A, (size_t)lda * 4, (size_t)K * 4, 1, s))))
      return rc; /* more rows cross below, in steps */
    a_dev = dA;
    a_ld = K;
    if (M == 1 && hipq::gemv_fuses_swiglu(w_act, w_mul, dA)) {
      if ((rc = hipq::launch_gemv_fused_swiglu(w_act, w_mul, dA, h_out ? h_out : dO, s))) return rc;
      if (h_out) return dio.finish();
      return stage_copy(false, dO, out, (size_t)ldo * 4, (size_t)N * 4, 1, s);
    }
  }
  const hipq_weight_t ws[2] = {w_act, w_mul};
  float *const cs[2] = {dY, dZ};
  const int64_t lds[2] = {N, N};
  if (mem == HIPQ_MEM_HOST && !h_out) { /* rows through the copy engines, in steps where that keeps the bits */
    bool keep = false;
    if ((rc = steps_keep_bits(2, ws, M, &keep))) return rc;
    RowSteps steps;
    if ((rc = steps.plan(s, M, keep, A, K, 1, &out, N))) return rc;
    for (int64_t r0 = 0; r0 < M;) {
      const int64_t n = steps.rows_at(r0);
      float *const cr[2] = {dY + r0 * N, dZ + r0 * N};
      if (M > 1 && (rc = steps.in(dA, A, lda, K, r0, n))) return rc;
      if ((rc = hipq_matmul_multi(2, ws, dA + r0 * K, n, K, cr, lds, HIPQ_MEM_DEVICE, stream))) return rc;
      if ((rc = hipq::launch_swiglu_rows(cr[0], cr[1], n, N, dO + r0 * N, N, s))) return rc;
      if ((rc = steps.out(dO, out, ldo, N, r0, n))) return rc;
      r0 += n;
    }
    return steps.finish();
  }
  if ((rc = hipq_matmul_multi(2, ws, a_dev, M, a_ld, cs, lds, HIPQ_MEM_DEVICE, stream))) return rc;
  if (mem == HIPQ_MEM_DEVICE) return hipq::launch_swiglu_rows(dY, dZ, M, N, out, ldo, s);
  if ((rc = hipq::launch_swiglu_rows(dY, dZ, M, N, h_out, h_ld, s))) return rc;
  return dio.finish();
}

int hipq_mlp_swiglu_down(hipq_weight_t w_act, hipq_weight_t w_mul, hipq_weight_t w_down, const float *A, int64_t M,
                         int64_t lda, float *out, int64_t ldo, int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!w_act || !w_mul || !w_down) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null weight");
  if ((rc = check_matmul_args(w_act, A, M, lda, out, w_act->N))) return rc;
  if ((rc = check_matmul_args(w_mul, A, M, lda, out, w_mul->N))) return rc;
  if (w_act->K != w_mul->K || w_act->N != w_mul->N)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the two projections differ in shape");
  if (w_down->K != w_act->N)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the down projection takes %lld values a row, the gated half gives %lld",
                (long long)w_down->K, (long long)w_act->N);
  if ((rc = check_matmul_args(w_down, A, M, w_down->K, out, ldo))) return rc;
  if (mem != HIPQ_MEM_DEVICE && mem != HIPQ_MEM_HOST)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  if (M == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);
  const int64_t N = w_act->N, K = w_act->K, Nd = w_down->N;
  /* one operand buffer for the whole call: the input rows (host operands), the two products, the hidden
   * rows and the output rows (host operands) */
  const size_t a_bytes = ((size_t)M * K * 4 + 255) & ~(size_t)255, h_bytes = ((size_t)M * N * 4 + 255) & ~(size_t)255,
               o_bytes = ((size_t)M * Nd * 4 + 255) & ~(size_t)255;
  void *io = nullptr;
  if ((rc = io_buffer(s, a_bytes + 3 * h_bytes + o_bytes, &io))) return rc;
  float *dA = (float *)io, *dY = (float *)((char *)io + a_bytes), *dZ = (float *)((char *)dY + h_bytes),
        *dH = (float *)((char *)dZ + h_bytes), *dO = (float *)((char *)dH + h_bytes);
  const float *a_dev = A;
  int64_t a_ld = lda;
  float *o_dev = out;
  int64_t o_ld = ldo;
  DirectIO dio;
  bool direct = false;
  if (mem == HIPQ_MEM_HOST) {
    if (dio.begin(s, A, M, lda, K, 1, &out, &ldo, &Nd, &rc)) { /* a decode step's rows: no copy engine */
      if ((rc = dio.fetch(dA, K))) return rc;
      o_dev = dio.outs[0].dev, o_ld = dio.outs[0].dld;
      direct = true;
    } else {
      if (rc) return rc;
      o_dev = dO, o_ld = Nd;
    }
    a_dev = dA, a_ld = K;
  }
  const hipq_weight_t ws[2] = {w_act, w_mul};
  const int64_t lds[2] = {N, N};
  /* rows [r0, r0 + n): the gated half into dH, the down projection into the output */
  auto rows = [&](int64_t r0, int64_t n) -> int {
    const float *a = a_dev + r0 * a_ld;
    int rr;
    if (n == 1 && hipq::gemv_fuses_swiglu(w_act, w_mul, a)) {
      if ((rr = hipq::launch_gemv_fused_swiglu(w_act, w_mul, a, dH + r0 * N, s))) return rr;
    } else {
      float *const cr[2] = {dY + r0 * N, dZ + r0 * N};
      if ((rr = hipq_matmul_multi(2, ws, a, n, a_ld, cr, lds, HIPQ_MEM_DEVICE, stream))) return rr;
      if ((rr = hipq::launch_swiglu_rows(cr[0], cr[1], n, N, dH + r0 * N, N, s))) return rr;
    }
    return hipq_matmul(w_down, dH + r0 * N, n, N, o_dev + r0 * o_ld, o_ld, HIPQ_MEM_DEVICE, stream);
  };
  if (mem == HIPQ_MEM_DEVICE || direct) {
    if ((rc = rows(0, M))) return rc;
    return direct ? dio.finish() : HIPQ_OK;
  }
  /* host rows through the copy engines, in steps where that keeps the bits */
  const hipq_weight_t all[3] = {w_act, w_mul, w_down};
  bool keep = false;
  if ((rc = steps_keep_bits(3, all, M, &keep))) return rc;
  RowSteps steps;
  if ((rc = steps.plan(s, M, keep, A, K, 1, &out, Nd))) return rc;
  for (int64_t r0 = 0; r0 < M;) {
    const int64_t n = steps.rows_at(r0);
    if ((rc = steps.in(dA, A, lda, K, r0, n))) return rc;
    if ((rc = rows(r0, n))) return rc;
    if ((rc = steps.out(dO, out, ldo, Nd, r0, n))) return rc;
    r0 += n;
  }
  return steps.finish();
}

int hipq_matmul_multi(int count, const hipq_weight_t *w, const float *A, int64_t M, int64_t lda,
                      float *const *C, const int64_t *ldc, int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (count <= 0 || !w || !C || !ldc) return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad weight list");
  for (int i = 0; i < count; ++i) {
    if ((rc = check_matmul_args(w[i], A, M, lda, C[i], ldc[i]))) return rc;
    if (w[i]->K != w[0]->K) return fail(HIPQ_ERR_INVALID_ARGUMENT, "weights disagree on K");
  }
  if (mem != HIPQ_MEM_DEVICE && mem != HIPQ_MEM_HOST)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  if (M == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);
  if (mem == HIPQ_MEM_HOST) {
    /* the activation crosses once, the products run as for device memory, the outputs return */
    const int64_t Kh = w[0]->K;
    size_t total = ((size_t)M * Kh * 4 + 255) & ~(size_t)255;
    std::vector<size_t> off(count);
    for (int i = 0; i < count; ++i) {
      off[i] = total;
      total += ((size_t)M * w[i]->N * 4 + 255) & ~(size_t)255;
    }
    void *io = nullptr;
    if ((rc = io_buffer(s, total, &io))) return rc;
    std::vector<float *> dC(count);
    std::vector<int64_t> dld(count);
    /* a decode step's rows: fetched by a kernel, the outputs written by the product kernels */
    DirectIO dio;
    std::vector<int64_t> ns(count);
    for (int i = 0; i < count; ++i) ns[i] = w[i]->N;
    if (dio.begin(s, A, M, lda, Kh, count, C, ldc, ns.data(), &rc)) {
      for (int i = 0; i < count; ++i) dC[i] = dio.outs[i].dev, dld[i] = dio.outs[i].dld;
      if ((rc = dio.fetch((float *)io, Kh))) return rc;
      if ((rc = hipq_matmul_multi(count, w, (const float *)io, M, Kh, dC.data(), dld.data(), HIPQ_MEM_DEVICE, stream)))
        return rc;
      return dio.finish();
    }
    if (rc) return rc;
    for (int i = 0; i < count; ++i) {
      dC[i] = (float *)((char *)io + off[i]);
      dld[i] = w[i]->N;
    }
    /* rows through the copy engines, in steps where that keeps the bits */
    bool keep = false;
    if ((rc = steps_keep_bits(count, w, M, &keep))) return rc;
    RowSteps steps;
    int64_t out_cols = 0;
    for (int i = 0; i < count; ++i) out_cols += w[i]->N;
    if ((rc = steps.plan(s, M, keep, A, Kh, count, C, out_cols))) return rc;
    std::vector<float *> dCr(count);
    for (int64_t r0 = 0; r0 < M;) {
      const int64_t n = steps.rows_at(r0);
      if ((rc = steps.in((float *)io, A, lda, Kh, r0, n))) return rc;
      for (int i = 0; i < count; ++i) dCr[i] = dC[i] + r0 * dld[i];
      if ((rc = hipq_matmul_multi(count, w, (const float *)io + r0 * Kh, n, Kh, dCr.data(), dld.data(), HIPQ_MEM_DEVICE,
                                  stream)))
        return rc;
      for (int i = 0; i < count; ++i)
        if ((rc = steps.out(dC[i], C[i], ldc[i], w[i]->N, r0, n, i == 0))) return rc;
      r0 += n;
    }
    return steps.finish();
  }
  if (M == 1 && hipq::gemv_fuses_quantizer_multi(count, w, A))
    return hipq::launch_gemv_fused_multi(count, w, A, C, s);
  /* ONE reservation for the whole call, before anything is quantized: the largest scratch any
   * member's product asks for (its quantized rows in the plane, row or tiled form, and behind the
   * tiled form the partial products of a product in parts of K, which depend on the weight's tile
   * copy: that is built first). Members of a group read the rows the group's first product
   * quantized, so the block must not be replaced between them; `gen` is checked before every
   * product that reuses them. */
  uint64_t gen = 0;
  {
    size_t need = 0;
    for (int i = 0; i < count; ++i) {
      const hipq_weight *x = w[i];
      size_t n = qact_bytes(x->dtype != HIPQ_Q4_0, M, x->K);
      if (x->dtype != HIPQ_Q4_0 && wants_tiled(x, M)) {
        if (!x->gt_base && (rc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(x)))) return rc;
        const size_t parts = x->dtype == HIPQ_Q4_K ? hipq::gemm_q4k_split_bytes(x, M) : hipq::gemm_q6k_split_bytes(x, M);
        const size_t tiled = ((qact_tiled_bytes(M, x->K) + 255) & ~(size_t)255) + parts;
        if (tiled > n) n = tiled;
      }
      if (n > need) need = n;
    }
    void *reserve = nullptr;
    if ((rc = workspace(s, need, &reserve))) return rc;
    gen = workspace_generation(s);
  }
  /* one quantization per distinct activation format among the weights */
  /* two or more Q4_K weights against a few rows: one launch of the few-rows kernel for up to four of
   * them, where the launch as a whole is wide enough */
  const hipq_weight *q4k[64];
  int n_q4k = 0;
  for (int i = 0; i < count && n_q4k < 64; ++i)
    if (w[i]->dtype == HIPQ_Q4_K) q4k[n_q4k++] = w[i];
  const bool q4k_rows_group = n_q4k >= 2 && n_q4k < 64 && hipq::gemm_rows_q4k_fits_multi(n_q4k, q4k, M);
  auto klass = [&](const hipq_weight *x) {
    if (x->dtype == HIPQ_Q4_0) return 0;
    if (x->dtype == HIPQ_Q4_K && q4k_rows_group) return 5;
    if (wants_rows(x, M, true)) return 5; /* a few rows of Q4_K on the matrix cores: the row form of the MoE kernels */
    if (wants_tiled(x, M)) return x->dtype == HIPQ_Q4_K ? 3 : 4; /* the two tiled forms differ in their rows' quantizer */
    return (x->dtype == HIPQ_Q4_K && M > 1) ? 1 : 2;
  };
  {
    const hipq_weight *gw[4];
    float *gc[4];
    int64_t gl[4];
    int ng = 0;
    bool first = true;
    QAct qa{};
    for (int i = 0; i <= count; ++i) {
      if (i < count && klass(w[i]) != 5) continue;
      if (i < count) {
        if (first) { /* the one quantization, in the row form of the matrix-core kernels */
          if ((rc = matmul_rows(w[i], A, M, lda, C[i], ldc[i], s, 2, Scratch{false, s}))) return rc;
          void *mem = nullptr;
          if ((rc = workspace(s, qact_bytes(1, M, w[i]->K), &mem))) return rc;
          qa = qact_carve(1, mem, M, w[i]->K);
          first = false;
        }
        if (!w[i]->gt_base && (rc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(w[i])))) return rc;
        gw[ng] = w[i], gc[ng] = C[i], gl[ng] = ldc[i];
        ++ng;
      }
      if (ng == 4 || (i == count && ng)) {
        if ((rc = workspace_unmoved(s, gen))) return rc;
        if ((rc = hipq::launch_gemm_rows_q4k_multi(ng, gw, &qa, (int)M, (int)((M / 4) * 4), gc, gl, s))) return rc;
        ng = 0;
      }
    }
  }
  for (int k = 3; k <= 4; ++k) {
    int members = 0;
    for (int i = 0; i < count; ++i) members += klass(w[i]) == k;
    if (k == 3 && members > 1) {
      /* Q4_K: one quantization, then the products four weights a launch (the grids of K and V of
       * a layer with grouped-query attention would be an eighth of the chip each) */
      void *mem = nullptr;
      if ((rc = workspace(s, qact_tiled_bytes(M, w[0]->K), &mem))) return rc;
      const QActTiled qa = qact_tiled_carve(mem, M, w[0]->K);
      if ((rc = hipq::launch_quantize_q8_K_tiled(A, M, w[0]->K, lda, (M / 4) * 4, &qa, s))) return rc;
      const hipq_weight *gw[4];
      float *gc[4];
      int64_t gl[4];
      int ng = 0;
      for (int i = 0; i < count; ++i) {
        if (klass(w[i]) != k) continue;
        if (!w[i]->gt_base && (rc = hipq::ensure_gemm_tiles(const_cast<hipq_weight *>(w[i])))) return rc;
        gw[ng] = w[i], gc[ng] = C[i], gl[ng] = ldc[i];
        if (++ng == 4) {
          if ((rc = workspace_unmoved(s, gen))) return rc;
          if ((rc = hipq::launch_gemm_q4k_multi(ng, gw, &qa, (int)M, gc, gl, s))) return rc;
          ng = 0;
        }
      }
      if (ng && (rc = workspace_unmoved(s, gen))) return rc;
      if (ng && (rc = hipq::launch_gemm_q4k_multi(ng, gw, &qa, (int)M, gc, gl, s))) return rc;
      continue;
    }
    bool first = true;
    for (int i = 0; i < count; ++i)
      if (klass(w[i]) == k) {
        /* the products after the first read the rows the first one quantized */
        if (!first && (rc = workspace_unmoved(s, gen))) return rc;
        if ((rc = matmul_tiled(w[i], A, M, lda, C[i], ldc[i], s, first ? 0 : 1, Scratch{false, s}))) return rc;
        first = false;
      }
  }
  for (int k = 0; k < 3; ++k) {
    int first = -1;
    for (int i = 0; i < count; ++i)
      if (klass(w[i]) == k) {
        first = i;
        break;
      }
    if (first < 0) continue;
    const int is_k = k != 0;
    if (k == 0) { /* up to four Q4_0 weights and a few rows: one launch that quantizes the rows itself */
      const hipq_weight *fw[4];
      float *fc[4];
      int64_t fl[4];
      int nf = 0, members = 0;
      for (int i = 0; i < count; ++i)
        if (klass(w[i]) == 0) {
          if (nf < 4) fw[nf] = w[i], fc[nf] = C[i], fl[nf] = ldc[i], ++nf;
          ++members;
        }
      if (members <= 4 && hipq::gemm_rows_q40_fuses(nf, fw, M, A, lda)) {
        if ((rc = hipq::launch_gemm_rows_q40_fused(nf, fw, A, lda, (int)M, fc, fl, s))) return rc;
        continue;
      }
    }
    void *memp = nullptr;
    if ((rc = workspace(s, qact_bytes(is_k, M, w[0]->K), &memp))) return rc;
    QAct qa = qact_carve(is_k, memp, M, w[0]->K);
    if ((rc = quantize_for(w[first], A, M, lda, qa, s))) return rc;
    /* Q4_0 products go out four weights a launch (Q, K, V or gate, up: one grid that fills the
     * chip instead of three or two small ones): a few rows through the few-rows kernel where the
     * launch as a whole is wide enough for it, more than eight otherwise through the prefill GEMM */
    const hipq_weight *gw[4];
    float *gc[4];
    int64_t gl[4];
    int ng = 0;
    auto flush = [&]() -> int {
      int frc = workspace_unmoved(s, gen);
      if (frc) return frc;
      if (k == 0 && ng > 1 && hipq::gemm_rows_q40_fits_multi(ng, gw, M))
        frc = hipq::launch_gemm_rows_q40_multi(ng, gw, &qa, (int)M, gc, gl, s);
      else if (k == 0 && M > 8 && gw[0]->K % 256 == 0)
        frc = hipq::launch_gemm_multi(ng, gw, &qa, (int)M, gc, gl, s);
      else
        for (int j = 0; j < ng && !frc; ++j) frc = multiply(gw[j], qa, M, gc[j], gl[j], s);
      ng = 0;
      return frc;
    };
    for (int i = 0; i < count; ++i) {
      if (klass(w[i]) != k) continue;
      gw[ng] = w[i], gc[ng] = C[i], gl[ng] = ldc[i];
      if (++ng == 4 && (rc = flush())) return rc;
    }
    if (ng && (rc = flush())) return rc;
  }
  return HIPQ_OK;
}

/* ---- kernel timing ------------------------------------------------------------ */

int hipq_launch_timing_begin(int max_launches) {
  int rc = require_ready();
  if (rc) return rc;
  if (max_launches <= 0 || max_launches > (1 << 20)) return fail(HIPQ_ERR_INVALID_ARGUMENT, "max_launches = %d", max_launches);
  hipq::LaunchLog &lg = hipq::launch_log;
  if (lg.on) return fail(HIPQ_ERR_INVALID_ARGUMENT, "kernel timing is already on for this thread");
  while (lg.ev.size() < (size_t)2 * max_launches) {
    hipEvent_t e;
    HIPQ_HIP(hipEventCreate(&e));
    lg.ev.push_back(e);
  }
  lg.fn.assign((size_t)max_launches, nullptr);
  /* events beyond this call's limit stay in the pool but are not used */
  while (lg.ev.size() > (size_t)2 * max_launches) {
    (void)hipEventDestroy(lg.ev.back());
    lg.ev.pop_back();
  }
  lg.count = 0;
  lg.dropped = 0;
  lg.on = true;
  return HIPQ_OK;
}

int hipq_launch_timing_end(int capacity, int *count, float *ms, const char **names) {
  hipq::LaunchLog &lg = hipq::launch_log;
  if (!lg.on) return fail(HIPQ_ERR_INVALID_ARGUMENT, "kernel timing is not on for this thread");
  lg.on = false;
  if (!count || capacity < 0 || (capacity && !ms)) return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad argument");
  *count = lg.count;
  const int n = lg.count < capacity ? lg.count : capacity;
  for (int i = 0; i < n; ++i) {
    HIPQ_HIP(hipEventSynchronize(lg.ev[2 * i + 1]));
    HIPQ_HIP(hipEventElapsedTime(&ms[i], lg.ev[2 * i], lg.ev[2 * i + 1]));
    if (names) names[i] = lg.fn[i] ? lg.fn[i] : "";
  }
  if (lg.dropped)
    return fail(HIPQ_ERR_NOT_SUPPORTED, "%d launches beyond the %d the timing was opened for were not timed", lg.dropped,
                (int)lg.fn.size());
  return HIPQ_OK;
}

/* ---- mixture of experts ---------------------------------------------------- */

int hipq_moe_forward(const hipq_moe_desc *desc, const hipq_weight_t *gate, const hipq_weight_t *up,
                     const hipq_weight_t *down, const float *x, const float *router_logits,
                     const float *router_weight, float *y, int32_t *topk_idx, float *topk_w,
                     int mem, void *stream) {
  return hipq_moe_forward_ext(desc, nullptr, gate, up, down, x, router_logits, router_weight, y, topk_idx,
                              topk_w, mem, stream);
}

int hipq_moe_forward_ext(const hipq_moe_desc *desc, const hipq_moe_ext *ext, const hipq_weight_t *gate,
                         const hipq_weight_t *up, const hipq_weight_t *down, const float *x,
                         const float *router_logits, const float *router_weight, float *y,
                         int32_t *topk_idx, float *topk_w, int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!desc || !gate || !up || !down || !x || !y)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  const hipq_moe_desc d = *desc;
  hipq_moe_ext x_ = {};
  if (ext) x_ = *ext;
  if (x_.variant != HIPQ_MOE_QWEN && x_.variant != HIPQ_MOE_GPT_OSS)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown MoE variant %d", x_.variant);
  if (x_.variant == HIPQ_MOE_GPT_OSS && (!x_.gate_bias || !x_.up_bias || !x_.down_bias))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "the gpt_oss variant needs gate_bias, up_bias and down_bias");
  if (x_.router_bias && router_logits)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "router_bias applies to logits formed from router_weight only");
  if (d.tokens < 0 || d.hidden <= 0 || d.intermediate <= 0 || d.experts <= 0 || d.topk <= 0 ||
      d.topk > d.experts || d.topk > 32 || d.experts > 1024)
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "bad MoE shape T=%d H=%d I=%d E=%d k=%d", d.tokens,
                d.hidden, d.intermediate, d.experts, d.topk);
  if ((router_logits == nullptr) == (router_weight == nullptr))
    return fail(HIPQ_ERR_INVALID_ARGUMENT, "pass exactly one of router_logits and router_weight");
  const int dt = gate[0] ? gate[0]->dtype : -1;
  for (int e = 0; e < d.experts; ++e) {
    if (!gate[e] || !up[e] || !down[e]) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null expert weight %d", e);
    if (gate[e]->dtype != dt || up[e]->dtype != dt || down[e]->dtype != dt)
      return fail(HIPQ_ERR_INVALID_ARGUMENT, "expert weights must share one dtype");
    if (gate[e]->N != d.intermediate || gate[e]->K != d.hidden || up[e]->N != d.intermediate ||
        up[e]->K != d.hidden || down[e]->N != d.hidden || down[e]->K != d.intermediate)
      return fail(HIPQ_ERR_INVALID_ARGUMENT, "expert %d weight dims do not match the block", e);
  }
  if (d.tokens == 0) return HIPQ_OK;
  hipStream_t s = (hipStream_t)stream;
  EnqueueGuard eg(enqueue_lock(s));
  CallScope call(s);

  /* device table of the 3E weight views, rebuilt only when the handles change; moe_mu keeps
   * the table from being rebuilt or freed by another thread before the launches below are in
   * the stream (whoever frees one synchronizes the device first, under the same lock) */
  WView *dev_views = nullptr;
  std::lock_guard<std::mutex> ml(g.moe_mu);
  {
    std::lock_guard<std::mutex> lk(g.mu);
    MoeTable &t = g.moe_tables[gate[0]];
    std::vector<const hipq_weight *> key;
    key.reserve(3 * (size_t)d.experts);
    for (int e = 0; e < d.experts; ++e) key.push_back(gate[e]);
    for (int e = 0; e < d.experts; ++e) key.push_back(up[e]);
    for (int e = 0; e < d.experts; ++e) key.push_back(down[e]);
    if (t.key != key || !t.dev) {
      /* experts that run on the matrix cores are stored by 32-row tiles from here on */
      if (hipq::moe_wants_tiles(&d, dt))
        for (const hipq_weight *w : key)
          if (!w->expert_tiles && (rc = hipq::tile_expert_weight(const_cast<hipq_weight *>(w)))) return rc;
      std::vector<WView> host(key.size());
      for (size_t i = 0; i < key.size(); ++i) host[i] = wview(key[i]);
      if (t.dev) {
        HIPQ_HIP(hipDeviceSynchronize()); /* another stream may still read the old table */
        HIPQ_HIP(hipFree(t.dev));
        t.dev = nullptr;
      }
      HIPQ_HIP(hipMalloc((void **)&t.dev, host.size() * sizeof(WView)));
      HIPQ_HIP(hipMemcpy(t.dev, host.data(), host.size() * sizeof(WView), hipMemcpyHostToDevice));
      t.key = key;
    }
    dev_views = t.dev;
  }

  const size_t ws_bytes = hipq::moe_workspace_bytes(&d);
  void *ws = nullptr;
  if ((rc = workspace(s, ws_bytes, &ws))) return rc;

  hipq::MoeArgs a;
  a.desc = d;
  a.gate = gate;
  a.up = up;
  a.down = down;
  a.epi.kind = x_.variant;
  a.epi.alpha = x_.alpha;
  a.epi.limit = x_.variant == HIPQ_MOE_GPT_OSS ? x_.limit : 0.f;
  a.epi.gate_bias = x_.gate_bias;
  a.epi.up_bias = x_.up_bias;
  a.epi.down_bias = x_.down_bias;
  a.router_bias = x_.router_bias;
  const size_t T = (size_t)d.tokens, H = (size_t)d.hidden, E = (size_t)d.experts, k = (size_t)d.topk;
  const size_t I = (size_t)d.intermediate;
  if (mem == HIPQ_MEM_DEVICE) {
    a.x = x;
    a.router_logits = router_logits;
    a.router_weight = router_weight;
    a.y = y;
    a.topk_idx = topk_idx;
    a.topk_w = topk_w;
    return hipq::launch_moe(&a, ws, ws_bytes, dev_views, s);
  }
  if (mem != HIPQ_MEM_HOST) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  /* host operands: device copies in the stream's operand buffer (no allocation per call); biases
   * and a router weight the caller keeps on the device are used where they are; a decode step's
   * few rows take no copy engine (DirectIO) */
  const bool gpt = x_.variant == HIPQ_MOE_GPT_OSS;
  const bool host_biases = !x_.biases_on_device;
  const bool host_router = router_logits || !x_.router_on_device;
  auto up256 = [](size_t n) { return (n + 255) & ~(size_t)255; };
  const size_t n_router = router_logits ? T * E : H * E;
  const size_t o_x = 0, o_r = o_x + up256(T * H * 4), o_y = o_r + (host_router ? up256(n_router * 4) : 0),
               o_i = o_y + up256(T * H * 4), o_w = o_i + up256(T * k * 4), o_br = o_w + up256(T * k * 4),
               o_bg = o_br + (host_biases && x_.router_bias ? up256(E * 4) : 0),
               o_bu = o_bg + (host_biases && gpt ? up256(E * I * 4) : 0),
               o_bd = o_bu + (host_biases && gpt ? up256(E * I * 4) : 0),
               total = o_bd + (host_biases && gpt ? up256(E * H * 4) : 0);
  void *io = nullptr;
  if ((rc = io_buffer(s, total, &io))) return rc;
  char *base = (char *)io;
  if (host_biases) {
    if (x_.router_bias) {
      if ((rc = stage_copy(true, base + o_br, (void *)x_.router_bias, E * 4, E * 4, 1, s))) return rc;
      a.router_bias = (const float *)(base + o_br);
    }
    if (gpt) {
      if ((rc = stage_copy(true, base + o_bg, (void *)x_.gate_bias, I * 4, I * 4, E, s))) return rc;
      if ((rc = stage_copy(true, base + o_bu, (void *)x_.up_bias, I * 4, I * 4, E, s))) return rc;
      if ((rc = stage_copy(true, base + o_bd, (void *)x_.down_bias, H * 4, H * 4, E, s))) return rc;
      a.epi.gate_bias = (const float *)(base + o_bg);
      a.epi.up_bias = (const float *)(base + o_bu);
      a.epi.down_bias = (const float *)(base + o_bd);
    }
  }
  /* logits [T x E] or the router weight [H x E] */
  if (host_router) {
    if ((rc = stage_copy(true, base + o_r, (void *)(router_logits ? router_logits : router_weight), E * 4, E * 4,
                         router_logits ? T : H, s)))
      return rc;
    a.router_logits = router_logits ? (const float *)(base + o_r) : nullptr;
    a.router_weight = router_weight ? (const float *)(base + o_r) : nullptr;
  } else {
    a.router_logits = nullptr;
    a.router_weight = router_weight;
  }
  a.x = (const float *)(base + o_x);
  a.topk_idx = (int32_t *)(base + o_i);
  a.topk_w = (float *)(base + o_w);
  DirectIO dio;
  const int64_t h64 = (int64_t)H;
  if (!topk_idx && !topk_w && dio.begin(s, x, (int64_t)T, h64, h64, 1, &y, &h64, &h64, &rc)) {
    if ((rc = dio.fetch((float *)(base + o_x), h64))) return rc;
    a.y = dio.outs[0].dev;
    if (dio.outs[0].dld != h64) return fail(HIPQ_ERR_RUNTIME, "internal: strided output of a decode step's MoE block");
    if ((rc = hipq::launch_moe(&a, ws, ws_bytes, dev_views, s))) return rc;
    return dio.finish();
  }
  if (rc) return rc;
  if ((rc = stage_copy(true, base + o_x, (void *)x, H * 4, H * 4, T, s))) return rc;
  a.y = (float *)(base + o_y);
  if ((rc = hipq::launch_moe(&a, ws, ws_bytes, dev_views, s))) return rc;
  if ((rc = stage_copy(false, base + o_y, y, H * 4, H * 4, T, s))) return rc;
  if (topk_idx && (rc = stage_copy(false, base + o_i, topk_idx, k * 4, k * 4, T, s))) return rc;
  if (topk_w && (rc = stage_copy(false, base + o_w, topk_w, k * 4, k * 4, T, s))) return rc;
  return HIPQ_OK;
}

/* ---- device memory for callers without a HIP runtime of their own ------------ */

int hipq_device_alloc(void **ptr, size_t bytes) {
  int rc = require_ready();
  if (rc) return rc;
  if (!ptr) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  *ptr = nullptr;
  hipError_t e = hipMalloc(ptr, bytes ? bytes : 16);
  if (e != hipSuccess) {
    *ptr = nullptr;
    return fail(HIPQ_ERR_OUT_OF_MEMORY, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  }
  return HIPQ_OK;
}

int hipq_device_free(void *ptr) {
  if (!ptr) return HIPQ_OK;
  int rc = require_ready();
  if (rc) return rc;
  HIPQ_HIP(hipFree(ptr)); /* waits for the device's work that may still read it */
  return HIPQ_OK;
}

int hipq_device_upload(void *dst_device, const void *src_host, size_t bytes, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!dst_device || !src_host) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  if ((rc = stage_copy(true, dst_device, (void *)src_host, bytes, bytes, 1, (hipStream_t)stream))) return rc;
  HIPQ_HIP(hipStreamSynchronize((hipStream_t)stream)); /* page-locked sources are read by the DMA engine later */
  return HIPQ_OK;
}

int hipq_device_download(void *dst_host, const void *src_device, size_t bytes, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!dst_host || !src_device) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  return stage_copy(false, (void *)src_device, dst_host, bytes, bytes, 1, (hipStream_t)stream);
}

/* ---- offline weight quantizers ---------------------------------------------- */

int hipq_quantize_weights(int dtype, const float *W, int64_t N, int64_t K, void *out_blocks,
                          int mem, void *stream) {
  int rc = require_ready();
  if (rc) return rc;
  if (!W || !out_blocks) return fail(HIPQ_ERR_INVALID_ARGUMENT, "null argument");
  const int64_t nbytes = hipq_weight_nbytes(dtype, N, K);
  if (nbytes < 0) return (int)nbytes;
  hipStream_t s = (hipStream_t)stream;
  if (mem == HIPQ_MEM_DEVICE) return hipq::launch_quantize_weights(dtype, W, N, K, out_blocks, s);
  if (mem != HIPQ_MEM_HOST) return fail(HIPQ_ERR_INVALID_ARGUMENT, "unknown mem kind %d", mem);
  DevBuf dW, dOut;
  if ((rc = dW.alloc((size_t)N * K * 4))) return rc;
  if ((rc = dOut.alloc((size_t)nbytes))) return rc;
  HIPQ_HIP(hipMemcpy(dW.p, W, (size_t)N * K * 4, hipMemcpyHostToDevice));
  if ((rc = hipq::launch_quantize_weights(dtype, (const float *)dW.p, N, K, dOut.p, s))) return rc;
  HIPQ_HIP(hipStreamSynchronize(s));
  HIPQ_HIP(hipMemcpy(out_blocks, dOut.p, (size_t)nbytes, hipMemcpyDeviceToHost));
  return HIPQ_OK;
}

} /* extern "C" */
