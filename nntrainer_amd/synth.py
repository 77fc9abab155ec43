"""Bit-reproducible synthetic inputs (fp32 normals, token ids) for tests and bench.

Thin ctypes wrapper over csrc/synth.c: a counter-based generator whose normals use
only IEEE + - * / sqrt, so the same (seed, shape) gives the same bits everywhere.
"""
import ctypes as C
import hashlib
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "lib", "libhipq_synth.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            raise FileNotFoundError("%s is missing: run `make -C %s`" % (_PATH, os.path.join(_HERE, "csrc")))
        _lib = C.CDLL(_PATH)
        _lib.synth_normal.argtypes = [C.c_uint64, C.c_uint64, C.c_int64, C.c_double, C.c_void_p]
        _lib.synth_uniform_int.argtypes = [C.c_uint64, C.c_uint64, C.c_int64, C.c_int32, C.c_void_p]
    return _lib


def normal(seed, shape, sigma=1.0, first=0):
    """fp32 array of `shape`, N(0, sigma^2), stream `seed` starting at sample `first`."""
    out = np.empty(shape, np.float32)
    _load().synth_normal(seed, first, out.size, float(sigma), out.ctypes.data)
    return out


def token_ids(seed, n, vocab):
    out = np.empty(n, np.int32)
    _load().synth_uniform_int(seed, 0, n, vocab, out.ctypes.data)
    return out


def digest(a):
    """Short hash of an array's bytes, to tell input drift from kernel bugs."""
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:16]
