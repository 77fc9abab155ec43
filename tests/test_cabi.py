"""CPU: the C-ABI library loads, exports every symbol include/hipq.h declares, and
fails loudly (no fallback) where there is no GPU."""
import os
import re

import pytest

from nntrainer_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "hipq.h")).read()
    return sorted(set(re.findall(r"HIPQ_API\s+[\w\s\*]+?\b(hipq_\w+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = _declared()
    assert len(names) >= 15 and set(names) == set(capi.SYMBOLS)
    lib = capi.lib()
    for n in names:
        assert getattr(lib, n) is not None


def test_product_library_exports_exactly_the_header(tmp_path):
    """libhipq.so exports the functions include/hipq.h declares and no others; the measurement
    and test helpers live in libhipq_bench.so, which links it."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if " T " in line)
    assert exported == _declared(), set(exported) ^ set(_declared())
    bench = os.path.join(os.path.dirname(capi.LIB_PATH), "libhipq_bench.so")
    out = subprocess.run(["nm", "-D", "--defined-only", bench], capture_output=True, text=True, check=True).stdout
    have = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert set(capi.BENCH_SYMBOLS) <= have
    needed = subprocess.run(["readelf", "-d", bench], capture_output=True, text=True, check=True).stdout
    assert "libhipq.so" in needed


def test_weight_size_rules():
    # 18 B / 32, 144 B / 256, 210 B / 256 (q4_0_tensor.h:20-31, q4_k_tensor.h:25-33, q6_k_tensor.h:25-32)
    assert capi.weight_nbytes("q4_0", 4096, 4096) == 9437184
    assert capi.weight_nbytes("q4_K", 12288, 4096) == 28311552
    assert capi.weight_nbytes("q6_K", 151936, 4096) == 510504960
    for kind, k in (("q4_0", 48), ("q4_K", 128), ("q6_K", 300)):
        with pytest.raises(capi.HipqError) as e:
            capi.weight_nbytes(kind, 8, k)
        assert e.value.code == -1


def test_model_file_offsets_follow_the_reference_rule():
    """MODEL_FORMAT_BIN is the graph's tensors back to back; only tensors with
    quantization parameters other than Q4_0 / Q6_K carry a 16-bit scheme word in front
    (models/neuralnet.cpp:696-703). Host arithmetic: no device needed."""
    tensors = [("skip", 151936 * 1024 * 4),            # fp32 embedding
               ("skip", 1024 * 4),                     # a norm's gamma
               ("q4_0", 2048, 1024, capi.LAYOUT_X8),
               ("q4_K", 3072, 1024, capi.LAYOUT_X8),
               ("q4_K", 1024, 3072, capi.LAYOUT_X8),
               ("q6_K", 151936, 1024)]
    offs, end = capi.file_layout(tensors, offset=16)
    want, at = [], 16
    for t in tensors:
        if t[0] == "skip":
            want.append(at)
            at += t[1]
            continue
        if t[0] == "q4_K":
            at += 2
        want.append(at)
        at += capi.weight_nbytes(t[0], t[1], t[2])
    assert offs == want and end == at
    assert capi.file_layout([], offset=5) == ([], 5)
    with pytest.raises(capi.HipqError):
        capi.file_layout([("q4_K", 8, 100)])
    with pytest.raises(capi.HipqError):
        capi.file_layout([("skip", -1)])


def test_no_gpu_means_loud_failure():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(capi.HipqError):
        capi.init(0)
    import numpy as np
    blocks = np.zeros(capi.weight_nbytes("q4_0", 8, 32), np.uint8)
    with pytest.raises(capi.HipqError) as e:
        capi.Weight("q4_0", 8, 32, blocks)
    assert e.value.code == -2  # HIPQ_ERR_NOT_INITIALIZED: nothing computes without the device
    with pytest.raises(capi.HipqError) as e:
        capi.weights_from_file("/nonexistent", [("q4_0", 8, 32)])
    assert e.value.code == -2


def test_product_never_imports_the_oracle():
    """The package and the library sources must not reach into oracle/."""
    for base, _, files in os.walk(os.path.join(ROOT, "nntrainer_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".c", ".cpp", "Makefile")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "oracle" not in text.lower().replace("oracle/_ref", ""), os.path.join(base, f)
