"""Host C++ layer: the HIP context plug-in and its layers, without a GPU.

The plug-in is built against this repo's stand-in of the framework API and
driven by nntrainer_amd/lib/hipq_host_selftest, which loads it the way the
framework's Engine::registerContext does (dlopen + ml_train_context_pluggable,
nntrainer/engine.cpp:140-171 in the reference checkout). Where the reference
checkout is present the same adapter sources are also compiled against the
framework's own headers."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "nntrainer_amd", "lib")
HOST = os.path.join(ROOT, "nntrainer_amd", "host")
PLUGIN = os.path.join(LIB, "libnntrainer_hip_context.so")
DRIVER = os.path.join(LIB, "hipq_host_selftest")
REFERENCE = "/root/reference"


def _built():
    if not (os.path.exists(PLUGIN) and os.path.exists(DRIVER)):
        pytest.skip("host plug-in not built (run __graft_entry__.build())")


def test_plugin_exports_context_record():
    _built()
    out = subprocess.run(["nm", "-D", "--defined-only", PLUGIN], capture_output=True, text=True, check=True).stdout
    assert "ml_train_context_pluggable" in out


def test_context_factory_properties_and_finalize():
    """Factory keys, error types, property parsing and requested tensors."""
    _built()
    r = subprocess.run([DRIVER, PLUGIN, "api"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "API CHECKS PASSED" in r.stdout


def test_forward_without_device_raises(tmp_path):
    """No CPU fallback: without a usable GPU a forward call is a runtime_error."""
    _built()
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import numpy as np
    k, n = 256, 8
    (tmp_path / "w.bin").write_bytes(bytes(n * k // 256 * 144))
    np.zeros((1, k), np.float32).tofile(tmp_path / "x.bin")
    r = subprocess.run([DRIVER, PLUGIN, "fc", "q4_K", str(k), str(n), "1", "1", "0", "0",
                        str(tmp_path / "w.bin"), str(tmp_path / "x.bin"), "-", str(tmp_path / "y.bin")],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 3, r.stdout + r.stderr
    assert "no usable HIP device" in r.stdout


ADAPTERS = ["hip_context.cpp", "hip_mem_allocator.cpp", "fc_layer_hip.cpp", "moe_layer_hip.cpp",
            "qkv_layer_hip.cpp", "tie_word_embedding_hip.cpp", "mlp_swiglu_layer_hip.cpp", "hipq_host.cpp"]


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="reference checkout not present")
@pytest.mark.parametrize("src", ADAPTERS)
def test_adapters_compile_against_framework_headers(src, tmp_path):
    """The adapter sources compile to object code against the framework's own headers, and what
    the objects leave undefined is only what the framework, this library, the C++ runtime and libc
    provide: nothing of the stand-in API leaks into a build inside the framework's tree."""
    dirs = ["nntrainer", "nntrainer/layers", "nntrainer/tensor", "nntrainer/utils", "nntrainer/graph",
            "nntrainer/models", "nntrainer/optimizers", "nntrainer/dataset", "nntrainer/compiler",
            "nntrainer/tensor/cpu_backend", "nntrainer/tensor/cpu_backend/x86",
            "nntrainer/tensor/cpu_backend/fallback", "nntrainer/tensor/cpu_backend/ggml_interface", "api",
            "api/ccapi/include"]
    obj = str(tmp_path / (src + ".o"))
    cmd = ["g++", "-std=c++17", "-O1", "-fPIC", "-c", "-DHIPQ_WITH_NNTRAINER", "-I" + os.path.join(ROOT, "include"),
           "-I" + HOST] + ["-I" + os.path.join(REFERENCE, d) for d in dirs] + [os.path.join(HOST, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]
    mangled = subprocess.run(["nm", "--undefined-only", obj], capture_output=True, text=True, timeout=60)
    pretty = subprocess.run(["nm", "-C", "--undefined-only", obj], capture_output=True, text=True, timeout=60)
    assert mangled.returncode == 0 and pretty.returncode == 0, mangled.stderr + pretty.stderr
    import ctypes
    system = [ctypes.CDLL(n) for n in ("libc.so.6", "libstdc++.so.6", "libm.so.6", "libgcc_s.so.1")]
    framework = ("nntrainer::", "ml::train::", "causallm::", "__nntrainer_log_print")
    bad = []
    for raw, dem in zip(mangled.stdout.splitlines(), pretty.stdout.splitlines()):
        sym, name = raw.split()[-1], dem.split(None, 1)[1].strip()
        if sym.startswith("hipq_") or name.startswith("hipq_host::") or any(f in name for f in framework):
            continue  # this library (C ABI, host core); the framework
        if sym in ("_GLOBAL_OFFSET_TABLE_", "__dso_handle", "__tls_get_addr"):
            continue  # the linker's and the loader's
        if any(hasattr(lib, sym) for lib in system):
            continue  # libc, the C++ runtime, libm, the unwinder
        bad.append(name)
    assert not bad, bad
