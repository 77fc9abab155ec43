"""MI355X (gfx950) quantized-weight matmul back-end for NNTrainer's FC / MoE path.

The product is the C-ABI shared library ``nntrainer_amd/lib/libhipq.so`` declared in
``include/hipq.h`` (hand-written HIP kernels). This package holds its sources
(``csrc/``), the C++ host layer that plugs it into NNTrainer's Context / Layer
interface (``host/``) and a thin ctypes binding (``capi``) used by the tests and
the benchmark. There is no CPU fallback: without the built library or without a
gfx950 device every call raises.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
