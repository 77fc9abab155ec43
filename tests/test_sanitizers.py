"""CPU: the host code that is not GPU code -- the oracle and the framework plug-in with its
driver -- built with AddressSanitizer and UndefinedBehaviorSanitizer and run once. The plug-in's
weight cache, property parsing and tensor bookkeeping and the oracle's block indexing are the
places where an out-of-bounds access would otherwise go unnoticed (or skew a parity result)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ENV = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1:abort_on_error=0",
           UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")


def _make(directory, target="asan"):
    r = subprocess.run(["make", "-C", directory, target], capture_output=True, text=True, timeout=900)
    if r.returncode != 0 and "sanitize" in r.stderr and "cannot find" in r.stderr:
        pytest.skip("the sanitizer runtimes are not installed here")
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]


def test_oracle_under_sanitizers():
    _make(os.path.join(ROOT, "oracle"))
    r = subprocess.run([os.path.join(ROOT, "oracle", "asan", "oracle_selfcheck")], capture_output=True, text=True,
                       timeout=600, env=ENV)
    assert r.returncode == 0 and "ORACLE SELFCHECK PASSED" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-4000:]


def test_host_plugin_under_sanitizers(tmp_path):
    lib = os.path.join(ROOT, "nntrainer_amd", "lib")
    if not os.path.exists(os.path.join(lib, "libhipq.so")):
        pytest.skip("libhipq.so not built (run __graft_entry__.build())")
    _make(os.path.join(ROOT, "nntrainer_amd", "host"))
    driver, plugin = os.path.join(lib, "asan", "hipq_host_selftest"), os.path.join(lib, "asan", "libnntrainer_hip_context.so")
    r = subprocess.run([driver, plugin, "api"], capture_output=True, text=True, timeout=600, env=ENV)
    assert r.returncode == 0 and "API CHECKS PASSED" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-4000:]
    import torch
    if torch.cuda.is_available():
        return
    # the error path of a forward call without a device: exceptions cross the plug-in boundary
    import numpy as np
    k, n = 256, 8
    (tmp_path / "w.bin").write_bytes(bytes(n * k // 256 * 144))
    np.zeros((1, k), np.float32).tofile(tmp_path / "x.bin")
    r = subprocess.run([driver, plugin, "fc", "q4_K", str(k), str(n), "1", "1", "0", "0", str(tmp_path / "w.bin"),
                        str(tmp_path / "x.bin"), "-", str(tmp_path / "y.bin")], capture_output=True, text=True,
                       timeout=600, env=ENV)
    assert r.returncode == 3 and "no usable HIP device" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-4000:]
