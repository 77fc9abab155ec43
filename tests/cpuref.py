"""ctypes doors to the two CPU checkers used by the tests.

`oracle()` loads oracle/liboracle.so, this repository's C restatement of the
reference arithmetic; `ref()` loads oracle/_ref/libnntr_ref.so, the reference's own
sources compiled as they lie (None when that library has not been built).
Both are test infrastructure: nothing in the product imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

Q4_0_BYTES, Q8_0_BYTES, Q4_K_BYTES, Q6_K_BYTES, Q8_K_BYTES = 18, 34, 144, 210, 292
BLOCK_BYTES = {"q4_0": (18, 32), "q4_K": (144, 256), "q6_K": (210, 256)}

_c = ctypes
_vp, _i64, _i32, _f32p = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p


def _ptr(a):
    return _c.c_void_p(a.ctypes.data)


def _load(path):
    lib = _c.CDLL(path)
    return lib


_oracle = None
_ref = None
_ref_tried = False


def oracle():
    global _oracle
    if _oracle is None:
        so = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(so):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"])
        lib = _load(so)
        lib.orc_fp16_to_fp32.restype = _c.c_float
        lib.orc_fp16_to_fp32.argtypes = [_c.c_uint16]
        lib.orc_fp32_to_fp16.restype = _c.c_uint16
        lib.orc_fp32_to_fp16.argtypes = [_c.c_float]
        _oracle = lib
    return _oracle


def ref():
    """The reference library, or None if it is not built (no reference checkout)."""
    global _ref, _ref_tried
    if not _ref_tried:
        _ref_tried = True
        so = os.path.join(ORACLE_DIR, "_ref", "libnntr_ref.so")
        if os.path.exists(so):
            lib = _load(so)
            lib.ref_init()
            lib.ref_fp16_to_fp32.restype = _c.c_float
            lib.ref_fp16_to_fp32.argtypes = [_c.c_uint16]
            lib.ref_fp32_to_fp16.restype = _c.c_uint16
            lib.ref_fp32_to_fp16.argtypes = [_c.c_float]
            lib.ref_vec_dot_q6_K_q8_K.restype = _c.c_float
            _ref = lib
    return _ref


# ---------------------------------------------------------------- weights
def quantize_weights(lib, kind, w):
    """w fp32 [N, K] -> uint8 canonical blocks [N * K/blk * bytes]."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    nbytes, blk = BLOCK_BYTES[kind]
    out = np.zeros(n * (k // blk) * nbytes, np.uint8)
    if lib is oracle():
        getattr(lib, "orc_quantize_" + kind)(_ptr(w), _ptr(out), _i64(n), _i64(k))
    else:
        getattr(lib, "ref_quantize_" + kind)(_ptr(w), _ptr(out), _i64(n), _i64(k))
    return out


def dequantize(lib, kind, blocks, n_elems):
    y = np.zeros(n_elems, np.float32)
    blocks = np.ascontiguousarray(blocks)
    if lib is oracle():
        getattr(lib, "orc_dequantize_" + kind)(_ptr(blocks), _ptr(y), _i64(n_elems))
    else:
        getattr(lib, "ref_dequantize_row_" + kind)(_ptr(blocks), _ptr(y), _i64(n_elems))
    return y


def repack_x8(lib, kind, blocks, n, k):
    blocks = np.ascontiguousarray(blocks)
    out = np.zeros_like(blocks)
    if lib is oracle():
        rc = getattr(lib, "orc_repack_%s_x8" % kind)(_ptr(out), _ptr(blocks), _i64(n), _i64(k))
        assert rc == 0
    else:
        getattr(lib, "ref_repack_%s_x8" % kind)(
            _ptr(out), _ptr(blocks), _c.c_size_t(blocks.size), _c.c_uint(n), _c.c_uint(k))
    return out


def unpack_x8(kind, blocks, n, k):
    blocks = np.ascontiguousarray(blocks)
    out = np.zeros_like(blocks)
    rc = getattr(oracle(), "orc_unpack_%s_x8" % kind)(_ptr(out), _ptr(blocks), _i64(n), _i64(k))
    assert rc == 0
    return out


# ---------------------------------------------------------------- activations
def quantize_act(lib, kind, x, variant="row"):
    """x fp32 [M, K] -> canonical activation blocks uint8 [M, K/blk*bytes].

    kind 'q8_0' | 'q8_K'; variant 'row' (row quantizer) or 'mat' (content of the
    reference's 4-row quantizer). With the reference library 'mat' runs the real
    4-row routine on groups of 4 rows (M % 4 == 0) and returns its interleaved bytes.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    m, k = x.shape
    nbytes, blk = (34, 32) if kind == "q8_0" else (292, 256)
    rowbytes = (k // blk) * nbytes
    out = np.zeros((m, rowbytes), np.uint8)
    if lib is oracle():
        fn = {("q8_0", "row"): lib.orc_quantize_row_q8_0,
              ("q8_0", "mat"): lib.orc_quantize_row_q8_0,
              ("q8_K", "row"): lib.orc_quantize_row_q8_K,
              ("q8_K", "mat"): lib.orc_quantize_row_q8_K_mat}[(kind, variant)]
        for i in range(m):
            fn(_c.c_void_p(x[i].ctypes.data), _c.c_void_p(out[i].ctypes.data), _i64(k))
        return out
    if variant == "row":
        fn = lib.ref_quantize_row_q8_0 if kind == "q8_0" else lib.ref_quantize_row_q8_K
        for i in range(m):
            fn(_c.c_void_p(x[i].ctypes.data), _c.c_void_p(out[i].ctypes.data), _i64(k))
        return out
    assert m % 4 == 0
    fn = lib.ref_quantize_mat_q8_0_4x8 if kind == "q8_0" else lib.ref_quantize_mat_q8_K_4x8
    out = out.reshape(m // 4, 4 * rowbytes)
    for g in range(m // 4):
        fn(_c.c_void_p(x[4 * g].ctypes.data), _c.c_void_p(out[g].ctypes.data), _i64(k))
    return out


def interleave4(kind, rows4, k):
    """4 canonical rows (uint8 [4, rowbytes]) -> reference 4-row interleaved bytes."""
    rows4 = np.ascontiguousarray(rows4)
    out = np.zeros(rows4.size, np.uint8)
    fn = oracle().orc_interleave_q8_0x4 if kind == "q8_0" else oracle().orc_interleave_q8_Kx4
    fn(_ptr(rows4), _ptr(out), _i64(k))
    return out


# ---------------------------------------------------------------- matmul
def gemm(lib, kind, a, w_blocks, n):
    """a fp32 [M, K]; w_blocks canonical blocks of W^T [n, K] -> fp32 [M, n].

    With the reference library Q4_0/Q4_K weights are first put in the x8 layout
    its kernels expect (by the reference's own repack)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    m, k = a.shape
    c = np.zeros((m, n), np.float32)
    w_blocks = np.ascontiguousarray(w_blocks)
    if lib is oracle():
        getattr(lib, "orc_gemm_" + kind)(_i32(m), _i32(n), _i32(k), _ptr(a), _ptr(w_blocks), _ptr(c))
    else:
        b = w_blocks if kind == "q6_K" else repack_x8(lib, kind, w_blocks, n, k)
        getattr(lib, "ref_gemm_" + kind)(_c.c_uint(m), _c.c_uint(n), _c.c_uint(k), _ptr(a), _ptr(b), _ptr(c))
    return c


def prepack(lib, kind, w_blocks, n, k):
    """Weights in the form `gemm_prepacked` takes: as they are for the oracle, in the
    x8 layout (done once) for the reference library's Q4_0 / Q4_K kernels."""
    w_blocks = np.ascontiguousarray(w_blocks)
    if lib is oracle() or kind == "q6_K":
        return w_blocks
    return repack_x8(lib, kind, w_blocks, n, k)


def gemm_prepacked(lib, kind, a, packed, n):
    a = np.ascontiguousarray(a, dtype=np.float32)
    m, k = a.shape
    c = np.zeros((m, n), np.float32)
    if lib is oracle():
        getattr(lib, "orc_gemm_" + kind)(_i32(m), _i32(n), _i32(k), _ptr(a), _ptr(packed), _ptr(c))
    else:
        getattr(lib, "ref_gemm_" + kind)(_c.c_uint(m), _c.c_uint(n), _c.c_uint(k), _ptr(a), _ptr(packed), _ptr(c))
    return c


def moe_forward(x, logits, gate, up, down, topk, kind="q4_K", renormalize=True):
    """Oracle MoE block. gate/up/down: lists (len E) of canonical block arrays of `kind`."""
    lib = oracle()
    x = np.ascontiguousarray(x, np.float32)
    logits = np.ascontiguousarray(logits, np.float32)
    t, h = x.shape
    e = logits.shape[1]
    nbytes, blk = BLOCK_BYTES[kind]
    i = gate[0].size // ((h // blk) * nbytes)
    arr = lambda lst: (_c.c_void_p * e)(*[w.ctypes.data for w in lst])
    y = np.zeros((t, h), np.float32)
    idx = np.zeros((t, topk), np.int32)
    wt = np.zeros((t, topk), np.float32)
    lib.orc_moe_forward(_i32({"q4_0": 2, "q4_K": 12, "q6_K": 14}[kind]), _i32(1 if renormalize else 0), _i32(t),
                        _i32(h), _i32(i), _i32(e), _i32(topk), _ptr(x), _ptr(logits), arr(gate), arr(up),
                        arr(down), _ptr(y), _ptr(idx), _ptr(wt))
    return y, idx, wt


def moe_forward_gpt_oss(x, logits, gate, up, down, gate_bias, up_bias, down_bias, topk, alpha=1.702, kind="q4_K",
                        renormalize=True):
    """Oracle GPT-OSS MoE block; logits already hold the router bias. Biases [E, I], [E, I], [E, H]."""
    lib = oracle()
    x = np.ascontiguousarray(x, np.float32)
    logits = np.ascontiguousarray(logits, np.float32)
    gb, ub, db = (np.ascontiguousarray(b, np.float32) for b in (gate_bias, up_bias, down_bias))
    t, h = x.shape
    e = logits.shape[1]
    nbytes, blk = BLOCK_BYTES[kind]
    i = gate[0].size // ((h // blk) * nbytes)
    arr = lambda lst: (_c.c_void_p * e)(*[w.ctypes.data for w in lst])
    y = np.zeros((t, h), np.float32)
    idx = np.zeros((t, topk), np.int32)
    wt = np.zeros((t, topk), np.float32)
    lib.orc_moe_forward_gpt_oss(_i32({"q4_0": 2, "q4_K": 12, "q6_K": 14}[kind]), _i32(1 if renormalize else 0),
                                _i32(t), _i32(h), _i32(i), _i32(e), _i32(topk), _ptr(x), _ptr(logits), arr(gate),
                                arr(up), arr(down), _ptr(gb), _ptr(ub), _ptr(db), _c.c_float(alpha), _ptr(y),
                                _ptr(idx), _ptr(wt))
    return y, idx, wt


def swiglu(y, z):
    """Oracle of nntrainer::swiglu: (y / (1 + exp(-y))) * z in fp32."""
    lib = oracle()
    y = np.ascontiguousarray(y, np.float32)
    z = np.ascontiguousarray(z, np.float32)
    x = np.empty_like(y)
    lib.orc_swiglu(_c.c_int64(y.size), _ptr(x), _ptr(y), _ptr(z))
    return x


def swiglu_x86(lib, y, z, alpha=None):
    """nntrainer::swiglu as the x86 back-end evaluates it (approximate exponential): the oracle's
    restatement, or the reference library's own routine."""
    y = np.ascontiguousarray(y, np.float32)
    z = np.ascontiguousarray(z, np.float32)
    x = np.zeros_like(y)
    if lib is oracle():
        if alpha is None:
            lib.orc_swiglu_x86(_c.c_int64(y.size), _ptr(x), _ptr(y), _ptr(z))
        else:
            lib.orc_swiglu_alpha_x86(_c.c_int64(y.size), _ptr(x), _ptr(y), _ptr(z), _c.c_float(alpha))
    elif alpha is None:
        lib.ref_swiglu(_c.c_uint(y.size), _ptr(x), _ptr(y), _ptr(z))
    else:
        lib.ref_swiglu_alpha(_c.c_uint(y.size), _ptr(x), _ptr(y), _ptr(z), _c.c_float(alpha))
    return x


def moe_forward_cached(x, logits, gate, up, down, topk, kind="q4_K", gpt_oss=False, gate_bias=None, up_bias=None,
                       down_bias=None, alpha=1.702, limit=7.0):
    """Oracle of the cached layers (moe_cached_slim; gpt_oss_moe_slim_cached with gpt_oss=True):
    one product per expert over its tokens, swiglu by token count, GPT-OSS with its clamps."""
    lib = oracle()
    x = np.ascontiguousarray(x, np.float32)
    logits = np.ascontiguousarray(logits, np.float32)
    t, h = x.shape
    e = logits.shape[1]
    nbytes, blk = BLOCK_BYTES[kind]
    i = gate[0].size // ((h // blk) * nbytes)
    if gpt_oss:
        gb, ub, db = (np.ascontiguousarray(b, np.float32) for b in (gate_bias, up_bias, down_bias))
    else:
        gb = ub = db = np.zeros(1, np.float32)
    arr = lambda lst: (_c.c_void_p * e)(*[w.ctypes.data for w in lst])
    y = np.zeros((t, h), np.float32)
    idx = np.zeros((t, topk), np.int32)
    wt = np.zeros((t, topk), np.float32)
    lib.orc_moe_forward_cached(_i32({"q4_0": 2, "q4_K": 12, "q6_K": 14}[kind]), _i32(1 if gpt_oss else 0), _i32(t),
                               _i32(h), _i32(i), _i32(e), _i32(topk), _ptr(x), _ptr(logits), arr(gate), arr(up),
                               arr(down), _ptr(gb), _ptr(ub), _ptr(db), _c.c_float(alpha), _c.c_float(limit),
                               _ptr(y), _ptr(idx), _ptr(wt))
    return y, idx, wt


def router_logits(x, wr, topk, bias=None):
    """x . wr in fp32, as the layers form their router logits (input.dot(gate_weights),
    qwen_moe_layer.cpp:436). The order of the fp32 sums is the BLAS's there and the device's here,
    so a case must not sit on a routing tie: the softmax values of the last expert taken and the
    first one left out differ by far more than such rounding can move them."""
    x = np.ascontiguousarray(x, np.float32)
    wr = np.ascontiguousarray(wr, np.float32)
    logits = (x @ wr).astype(np.float32)
    if bias is not None:
        logits = (logits + np.asarray(bias, np.float32)).astype(np.float32)
    p = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
    p = np.sort(p / p.sum(1, keepdims=True), axis=1)[:, ::-1]
    assert (p[:, topk - 1] - p[:, topk] > 1e-4 * p[:, 0]).all(), "routing tie in the test case"
    return logits
