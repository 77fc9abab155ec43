"""ctypes binding of the libhipq C ABI (include/hipq.h).

Device buffers are passed as raw addresses (``tensor.data_ptr()``); torch is only
the allocator and stream provider of the callers, it is not imported here.
"""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libhipq.so")
CSRC = os.path.join(HERE, "csrc")

Q4_0, Q4_K, Q6_K = 2, 12, 14
LAYOUT_CANONICAL, LAYOUT_X8 = 0, 1
MEM_HOST, MEM_DEVICE = 0, 1
Q8K_ROW, Q8K_MAT = 0, 1
DTYPES = {"q4_0": Q4_0, "q4_K": Q4_K, "q6_K": Q6_K}

SYMBOLS = [
    "hipq_init", "hipq_shutdown", "hipq_last_error", "hipq_version", "hipq_weight_nbytes",
    "hipq_weight_create", "hipq_weight_destroy", "hipq_weight_dims", "hipq_quantize_q8_0",
    "hipq_quantize_q8_K", "hipq_matmul", "hipq_matmul_each_row", "hipq_matmul_noalloc", "hipq_matmul_multi", "hipq_moe_forward",
    "hipq_moe_forward_ext", "hipq_mlp_swiglu", "hipq_mlp_swiglu_down", "hipq_host_alloc", "hipq_host_free", "hipq_stream_release",
    "hipq_quantize_weights", "hipq_file_layout", "hipq_weights_from_file",
    "hipq_device_alloc", "hipq_device_free", "hipq_device_upload", "hipq_device_download",
    "hipq_launch_timing_begin", "hipq_launch_timing_end",
]
# measurement and test helpers of csrc/hipq_bench.h: a library of their own (libhipq_bench.so)
# that links the product library; not part of the product
BENCH_SYMBOLS = ["hipq_bench_matmul_loop", "hipq_bench_mfma_ceiling", "hipq_bench_hbm_read_ceiling",
                 "hipq_bench_tiled_bytes", "hipq_bench_quantize_tiled", "hipq_bench_last_error"]


class HipqError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("hipq error %d: %s" % (code, msg))
        self.code = code


class FileTensor(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("layout", C.c_int32), ("N", C.c_int64), ("K", C.c_int64),
                ("bytes", C.c_int64)]


FILE_SKIP = -1


class MoeDesc(C.Structure):
    _fields_ = [("tokens", C.c_int32), ("hidden", C.c_int32), ("intermediate", C.c_int32),
                ("experts", C.c_int32), ("topk", C.c_int32), ("renormalize", C.c_int32)]


class MoeExt(C.Structure):
    _fields_ = [("variant", C.c_int32), ("alpha", C.c_float), ("router_bias", C.c_void_p),
                ("gate_bias", C.c_void_p), ("up_bias", C.c_void_p), ("down_bias", C.c_void_p),
                ("limit", C.c_float), ("biases_on_device", C.c_int32), ("router_on_device", C.c_int32)]


MOE_QWEN, MOE_GPT_OSS = 0, 1


def build(force=False):
    """Compile libhipq.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    if force:
        subprocess.check_call(["make", "-C", CSRC, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", CSRC, "-j8"], stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib():
    """The loaded library. Fails loudly if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `make -C %s` (there is no fallback path)" % (LIB_PATH, CSRC))
        L = C.CDLL(LIB_PATH)
        vp, i64, i32 = C.c_void_p, C.c_int64, C.c_int
        L.hipq_last_error.restype = C.c_char_p
        L.hipq_version.restype = C.c_char_p
        L.hipq_init.argtypes = [i32]
        L.hipq_weight_nbytes.restype = i64
        L.hipq_weight_nbytes.argtypes = [i32, i64, i64]
        L.hipq_weight_create.argtypes = [i32, i32, i64, i64, vp, i32, C.POINTER(vp)]
        L.hipq_weight_destroy.argtypes = [vp]
        L.hipq_file_layout.argtypes = [i32, C.POINTER(FileTensor), i64, C.POINTER(i64), C.POINTER(i64)]
        L.hipq_weights_from_file.argtypes = [C.c_char_p, i64, i32, C.POINTER(FileTensor), C.POINTER(vp),
                                             C.POINTER(i64)]
        L.hipq_weight_dims.argtypes = [vp, C.POINTER(i32), C.POINTER(i64), C.POINTER(i64)]
        L.hipq_quantize_q8_0.argtypes = [vp, i64, i64, i64, vp, i32, vp]
        L.hipq_quantize_q8_K.argtypes = [vp, i64, i64, i64, i32, vp, i32, vp]
        L.hipq_matmul.argtypes = [vp, vp, i64, i64, vp, i64, i32, vp]
        L.hipq_matmul_each_row.argtypes = [vp, vp, i64, i64, vp, i64, i32, vp]
        L.hipq_matmul_noalloc.argtypes = [vp, vp, i64, i64, vp, i64, vp]
        L.hipq_matmul_multi.argtypes = [i32, C.POINTER(vp), vp, i64, i64, C.POINTER(vp),
                                        C.POINTER(i64), i32, vp]
        L.hipq_moe_forward.argtypes = [C.POINTER(MoeDesc), C.POINTER(vp), C.POINTER(vp),
                                       C.POINTER(vp), vp, vp, vp, vp, vp, vp, i32, vp]
        L.hipq_moe_forward_ext.argtypes = [C.POINTER(MoeDesc), C.POINTER(MoeExt), C.POINTER(vp), C.POINTER(vp),
                                           C.POINTER(vp), vp, vp, vp, vp, vp, vp, i32, vp]
        L.hipq_quantize_weights.argtypes = [i32, vp, i64, i64, vp, i32, vp]
        L.hipq_mlp_swiglu.argtypes = [vp, vp, vp, i64, i64, vp, i64, i32, vp]
        L.hipq_mlp_swiglu_down.argtypes = [vp, vp, vp, vp, i64, i64, vp, i64, i32, vp]
        L.hipq_host_alloc.argtypes = [C.POINTER(vp), C.c_size_t]
        L.hipq_host_free.argtypes = [vp]
        L.hipq_stream_release.argtypes = [vp]
        L.hipq_device_alloc.argtypes = [C.POINTER(vp), C.c_size_t]
        L.hipq_device_free.argtypes = [vp]
        L.hipq_device_upload.argtypes = [vp, vp, C.c_size_t, vp]
        L.hipq_device_download.argtypes = [vp, vp, C.c_size_t, vp]
        L.hipq_launch_timing_begin.argtypes = [i32]
        L.hipq_launch_timing_end.argtypes = [i32, C.POINTER(i32), C.POINTER(C.c_float), C.POINTER(C.c_char_p)]
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise HipqError(rc, lib().hipq_last_error().decode())


def init(device=0):
    check(lib().hipq_init(device))


def shutdown():
    check(lib().hipq_shutdown())


def _addr(x):
    """Address of a numpy array, a torch tensor, an int, or None."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return x.ctypes.data


class Weight:
    """Device-resident quantized weight matrix (W^T: N rows of K values)."""

    def __init__(self, dtype, n, k, blocks, layout=LAYOUT_CANONICAL, mem=MEM_HOST):
        self.dtype = DTYPES.get(dtype, dtype)
        self.n, self.k = n, k
        self._h = C.c_void_p()
        check(lib().hipq_weight_create(self.dtype, layout, n, k, _addr(blocks), mem, C.byref(self._h)))

    @property
    def handle(self):
        return self._h

    def destroy(self):
        if self._h:
            check(lib().hipq_weight_destroy(self._h))
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def _file_tensors(tensors):
    """tensors: ("skip", nbytes) or (dtype, n, k[, layout]) in the file's order."""
    arr = (FileTensor * len(tensors))()
    for i, t in enumerate(tensors):
        if t[0] == "skip":
            arr[i] = FileTensor(FILE_SKIP, 0, 0, 0, t[1])
        else:
            arr[i] = FileTensor(DTYPES.get(t[0], t[0]), t[3] if len(t) > 3 else LAYOUT_CANONICAL, t[1], t[2], 0)
    return arr


def file_layout(tensors, offset=0):
    """Data offset of every listed tensor of a MODEL_FORMAT_BIN file and the end offset."""
    arr = _file_tensors(tensors)
    offs = (C.c_int64 * len(tensors))()
    end = C.c_int64()
    check(lib().hipq_file_layout(len(tensors), arr, offset, offs, C.byref(end)))
    return list(offs), end.value


def weights_from_file(path, tensors, offset=0):
    """Weight objects (None for skipped tensors) read from a MODEL_FORMAT_BIN file, and the
    offset behind the last listed tensor."""
    arr = _file_tensors(tensors)
    hs = (C.c_void_p * len(tensors))()
    end = C.c_int64()
    check(lib().hipq_weights_from_file(str(path).encode(), offset, len(tensors), arr, hs, C.byref(end)))
    out = []
    for t, h in zip(tensors, hs):
        if t[0] == "skip":
            out.append(None)
            continue
        w = Weight.__new__(Weight)
        w.dtype, w.n, w.k, w._h = DTYPES.get(t[0], t[0]), t[1], t[2], C.c_void_p(h)
        out.append(w)
    return out, end.value


def weight_nbytes(dtype, n, k):
    r = lib().hipq_weight_nbytes(DTYPES.get(dtype, dtype), n, k)
    if r < 0:
        raise HipqError(int(r), lib().hipq_last_error().decode())
    return int(r)


def quantize_q8_0(a, m, k, out, lda=None, mem=MEM_DEVICE, stream=None):
    check(lib().hipq_quantize_q8_0(_addr(a), m, k, lda or k, _addr(out), mem, stream))


def quantize_q8_K(a, m, k, out, variant=Q8K_ROW, lda=None, mem=MEM_DEVICE, stream=None):
    check(lib().hipq_quantize_q8_K(_addr(a), m, k, lda or k, variant, _addr(out), mem, stream))


def matmul(w, a, m, c, lda=None, ldc=None, mem=MEM_DEVICE, stream=None):
    check(lib().hipq_matmul(w.handle, _addr(a), m, lda or w.k, _addr(c), ldc or w.n, mem, stream))


def matmul_each_row(w, a, rows, c, lda=None, ldc=None, mem=MEM_DEVICE, stream=None):
    """`rows` independent one-row products in one call (the bits of `rows` calls of matmul with m = 1)."""
    check(lib().hipq_matmul_each_row(w.handle, _addr(a), rows, lda or w.k, _addr(c), ldc or w.n, mem, stream))


def matmul_noalloc(w, a, m, c, lda=None, ldc=None, stream=None):
    """hipq_matmul on device buffers with the quantized activations in the library's
    fixed scratch array: no device allocation inside the call."""
    check(lib().hipq_matmul_noalloc(w.handle, _addr(a), m, lda or w.k, _addr(c), ldc or w.n, stream))


def matmul_multi(ws, a, m, cs, ldc=None, mem=MEM_DEVICE, stream=None, lda=None):
    n = len(ws)
    hs = (C.c_void_p * n)(*[w.handle.value for w in ws])
    cp = (C.c_void_p * n)(*[_addr(c) for c in cs])
    ld = (C.c_int64 * n)(*(ldc if ldc is not None else [w.n for w in ws]))
    check(lib().hipq_matmul_multi(n, hs, _addr(a), m, lda or ws[0].k, cp, ld, mem, stream))


def mlp_swiglu(w_act, w_mul, a, m, out, lda=None, ldo=None, mem=MEM_DEVICE, stream=None):
    """out = swiglu(a . w_act^T, a . w_mul^T): the gated half of a dense MLP in one call."""
    check(lib().hipq_mlp_swiglu(w_act.handle, w_mul.handle, _addr(a), m, lda or w_act.k, _addr(out),
                                ldo or w_act.n, mem, stream))


def mlp_swiglu_down(w_act, w_mul, w_down, a, m, out, lda=None, ldo=None, mem=MEM_DEVICE, stream=None):
    """out = swiglu(a . w_act^T, a . w_mul^T) . w_down^T: the gated MLP of a decoder layer in one call."""
    check(lib().hipq_mlp_swiglu_down(w_act.handle, w_mul.handle, w_down.handle, _addr(a), m, lda or w_act.k,
                                     _addr(out), ldo or w_down.n, mem, stream))


def quantize_weights(dtype, w, n, k, out, mem=MEM_DEVICE, stream=None):
    check(lib().hipq_quantize_weights(DTYPES.get(dtype, dtype), _addr(w), n, k, _addr(out), mem, stream))


class Experts:
    """The handle arrays of a block's expert weights, built once: a decode step is a few
    tens of microseconds, less than marshalling 3 x E handles per call would cost."""

    def __init__(self, gate, up, down):
        arr = lambda ws: (C.c_void_p * len(ws))(*[w.handle.value for w in ws])
        self.weights = (list(gate), list(up), list(down))  # keeps the handles alive
        self.gate, self.up, self.down = arr(gate), arr(up), arr(down)


def moe_forward(tokens, hidden, inter, experts, topk, gate, up, down, x, y, router_logits=None,
                router_weight=None, topk_idx=None, topk_w=None, renormalize=True, mem=MEM_DEVICE,
                stream=None):
    """gate / up / down: lists of E weights each, or gate = Experts(...) and up = down = None."""
    d = MoeDesc(tokens, hidden, inter, experts, topk, 1 if renormalize else 0)
    ex = gate if isinstance(gate, Experts) else Experts(gate, up, down)
    check(lib().hipq_moe_forward(C.byref(d), ex.gate, ex.up, ex.down, _addr(x),
                                 _addr(router_logits), _addr(router_weight), _addr(y),
                                 _addr(topk_idx), _addr(topk_w), mem, stream))


def moe_forward_gpt_oss(tokens, hidden, inter, experts, topk, gate, up, down, x, y, gate_bias, up_bias,
                        down_bias, alpha=1.702, router_logits=None, router_weight=None, router_bias=None,
                        topk_idx=None, topk_w=None, renormalize=True, mem=MEM_DEVICE, stream=None, limit=0.0,
                        biases_on_device=False):
    """The GPT-OSS block: biased router and projections, (g / (1 + exp(-alpha g))) * (u + 1);
    limit > 0: the cached layer's clamps on the biased gate and up values."""
    d = MoeDesc(tokens, hidden, inter, experts, topk, 1 if renormalize else 0)
    ext = MoeExt(MOE_GPT_OSS, alpha, _addr(router_bias), _addr(gate_bias), _addr(up_bias), _addr(down_bias),
                 limit, 1 if biases_on_device else 0, 0)
    ex = gate if isinstance(gate, Experts) else Experts(gate, up, down)
    check(lib().hipq_moe_forward_ext(C.byref(d), C.byref(ext), ex.gate, ex.up, ex.down, _addr(x),
                                     _addr(router_logits), _addr(router_weight), _addr(y),
                                     _addr(topk_idx), _addr(topk_w), mem, stream))


def host_alloc(nbytes):
    """Address of `nbytes` of zero-filled page-locked host memory (hipq_host_free releases it)."""
    p = C.c_void_p()
    check(lib().hipq_host_alloc(C.byref(p), nbytes))
    return p.value


def host_free(addr):
    check(lib().hipq_host_free(addr))


def stream_release(stream=None):
    check(lib().hipq_stream_release(stream))


_bench = None


def bench_lib():
    """libhipq_bench.so: measurement and test helpers beside the product library."""
    global _bench
    if _bench is None:
        lib()  # the helpers link the product library
        path = os.path.join(os.path.dirname(LIB_PATH), "libhipq_bench.so")
        if not os.path.exists(path):
            raise FileNotFoundError("%s is missing: build it with `make -C %s`" % (path, CSRC))
        B = C.CDLL(path)
        vp, i64, i32, fp = C.c_void_p, C.c_int64, C.c_int, C.POINTER(C.c_float)
        B.hipq_bench_last_error.restype = C.c_char_p
        B.hipq_bench_matmul_loop.argtypes = [i32, C.POINTER(vp), vp, i64, i64, vp, i64, i32, vp, fp]
        B.hipq_bench_mfma_ceiling.argtypes = [C.c_float, vp, fp, fp]
        B.hipq_bench_hbm_read_ceiling.argtypes = [i64, i32, i32, vp, fp]
        B.hipq_bench_tiled_bytes.argtypes = [i64, i64]
        B.hipq_bench_tiled_bytes.restype = i64
        B.hipq_bench_quantize_tiled.argtypes = [vp, i64, i64, i64, vp, vp]
        _bench = B
    return _bench


def _bcheck(rc):
    if rc != 0:
        raise HipqError(rc, bench_lib().hipq_bench_last_error().decode())


def matmul_loop(ws, a, m, c, iters, stream=None):
    """Average milliseconds per call of `iters` hipq_matmul calls rotating over `ws`, two HIP events
    on `stream` around the loop (after one untimed call per weight)."""
    n = len(ws)
    hs = (C.c_void_p * n)(*[w.handle.value for w in ws])
    ms = C.c_float()
    _bcheck(bench_lib().hipq_bench_matmul_loop(n, hs, _addr(a), m, ws[0].k, _addr(c), ws[0].n, iters, stream,
                                               C.byref(ms)))
    return ms.value


class LaunchTiming:
    """with LaunchTiming(n) as t: ...calls...; afterwards t.launches = [(kernel name, ms), ...] in
    launch order: the kernels' own durations (hipq_launch_timing_begin / _end)."""

    def __init__(self, max_launches):
        self.max = int(max_launches)
        self.launches = []

    def __enter__(self):
        check(lib().hipq_launch_timing_begin(self.max))
        return self

    def __exit__(self, *exc):
        n = C.c_int()
        ms = (C.c_float * self.max)()
        names = (C.c_char_p * self.max)()
        rc = lib().hipq_launch_timing_end(self.max, C.byref(n), ms, names)
        if exc[0] is None:
            check(rc)
        k = min(n.value, self.max)
        self.launches = [((names[i] or b"").decode(), ms[i]) for i in range(k)]
        return False

    @staticmethod
    def _demangle(names):
        mangled = sorted({n for n in names if n.startswith("_Z")})
        if not mangled:
            return {}
        try:
            out = subprocess.run(["c++filt"] + mangled, capture_output=True, text=True, timeout=30).stdout.splitlines()
            return dict(zip(mangled, out)) if len(out) == len(mangled) else {}
        except (OSError, subprocess.SubprocessError):
            return {}

    def by_kernel(self):
        """{short kernel name: (launches, mean ms)}; the short name drops arguments and namespaces."""
        acc = {}
        plain = self._demangle([n for n, _ in self.launches])
        for name, ms in self.launches:
            name = plain.get(name, name)
            if name.endswith(" [clone .kd]"):
                name = name[:-len(" [clone .kd]")]
            short = name.split("(")[0].replace("(anonymous namespace)::", "").replace("void ", "").strip()
            short = short.replace("hipq::", "")
            cnt, tot = acc.get(short, (0, 0.0))
            acc[short] = (cnt + 1, tot + ms)
        return {k: (c, t / c) for k, (c, t) in acc.items()}


def bench_tiled_bytes(m, k):
    n = bench_lib().hipq_bench_tiled_bytes(m, k)
    if n < 0:
        raise HipqError(int(n), "bad shape")
    return int(n)


def bench_quantize_tiled(a, m, k, out, lda=None, stream=None):
    """The tiled Q8_K form of device rows `a` into the device buffer `out` (bench_tiled_bytes)."""
    _bcheck(bench_lib().hipq_bench_quantize_tiled(_addr(a), m, k, lda if lda is not None else k, _addr(out), stream))


def bench_hbm_read_ceiling(nbytes=1 << 30, waves_per_simd=4, regions=1, stream=None):
    """TB/s of a kernel that only reads `nbytes` of device memory (the GEMV kernels' access pattern);
    regions > 1: that many buffers, one per launch, back to back, each read cold."""
    tbs = C.c_float()
    _bcheck(bench_lib().hipq_bench_hbm_read_ceiling(nbytes, regions, waves_per_simd, stream, C.byref(tbs)))
    return tbs.value


def bench_mfma_ceiling(target_ms=2.0, stream=None):
    """(TOP/s, GHz) of a kernel that issues nothing but the int8 matrix instruction."""
    tops, ghz = C.c_float(), C.c_float()
    _bcheck(bench_lib().hipq_bench_mfma_ceiling(target_ms, stream, C.byref(tops), C.byref(ghz)))
    return tops.value, ghz.value
