"""GPU parity through the framework-facing layers: fully_connected and qwen_moe
created from the HIP context plug-in, fed host tensors in the layouts the
framework holds them in (x8-repacked Q4_0 / Q4_K bytes, canonical Q6_K), checked
against the oracle. Reads like the reference's layer tests: build the layer from
properties, finalize, fill weights, forward, compare."""
import os
import subprocess

import numpy as np
import pytest

from nntrainer_amd import synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "nntrainer_amd", "lib")
PLUGIN = os.path.join(LIB, "libnntrainer_hip_context.so")
DRIVER = os.path.join(LIB, "hipq_host_selftest")
TOL = 1e-4  # max |got - ref| / max |ref|, the bound for fp32 outputs of this path


def _framework_bytes(cr, kind, w32, n, k):
    blocks = cr.quantize_weights(cr.oracle(), kind, w32)
    if kind == "q6_K":
        return blocks, blocks
    return blocks, cr.repack_x8(cr.oracle(), kind, blocks, n, k)


def _run(args):
    r = subprocess.run([DRIVER, PLUGIN] + [str(a) for a in args], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("kind,k,n,height,bias", [
    ("q4_0", 1024, 512, 1, False),   # decode GEMV
    ("q4_K", 1024, 768, 1, False),
    ("q6_K", 512, 1000, 1, False),   # N not a multiple of 8: lm_head-like
    ("q4_K", 2048, 1024, 37, False), # prefill GEMM with a ragged last tile
    ("q4_0", 512, 256, 12, True),    # bias add
])
def test_fc_forwarding(cr, tmp_path, kind, k, n, height, bias):
    w32 = synth.normal(7000 + n, (n, k), 0.02)
    blocks, fw = _framework_bytes(cr, kind, w32, n, k)
    x = synth.normal(7100 + k, (height, k))
    b = synth.normal(7200, (n,), 0.5) if bias else None
    fw.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    if bias:
        b.tofile(tmp_path / "b.bin")
    _run(["fc", kind, k, n, 1, height, 0, 0, tmp_path / "w.bin", tmp_path / "x.bin",
          (tmp_path / "b.bin") if bias else "-", tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(height, n)
    ref = cr.gemm(cr.oracle(), kind, x, blocks, n)
    if bias:
        ref = ref + b
    err = np.abs(got - ref).max() / np.abs(ref).max()
    assert err <= TOL, err


def test_fc_incremental_forwarding_prefill_then_decode(cr, tmp_path):
    """incremental_forwarding(from, to) computes rows [0, to - from) of each batch
    entry and leaves the rest of the output alone (fc_layer.cpp:239-304)."""
    kind, k, n, batch, height = "q4_K", 512, 256, 2, 16
    w32 = synth.normal(7300, (n, k), 0.02)
    blocks, fw = _framework_bytes(cr, kind, w32, n, k)
    x = synth.normal(7301, (batch, height, k))
    fw.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    for frm, to in ((0, 16), (0, 5), (16, 17)):
        _run(["fc", kind, k, n, batch, height, frm, to, tmp_path / "w.bin", tmp_path / "x.bin", "-",
              tmp_path / "y.bin"])
        got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, height, n)
        rows = to - frm
        for b in range(batch):
            # the reference's rule (fc_layer.cpp:268-270): the input of batch entry b starts at
            # b times the OUTPUT's feature length, which differs from the entry's own rows
            # when in_width != unit (here 512 != 256)
            xin = x.reshape(-1)[b * height * n:][:rows * k].reshape(rows, k)
            ref = cr.gemm(cr.oracle(), kind, xin, blocks, n)
            err = np.abs(got[b, :rows] - ref).max() / np.abs(ref).max()
            assert err <= TOL, (frm, to, b, err)
            assert np.all(got[b, rows:] == -12345.0)


def test_fc_decode_row_is_bit_identical_to_oracle(cr, tmp_path):
    """M = 1 goes through the GEMV engine, which reproduces the reference's fp32
    evaluation order: equal bits, not just within tolerance."""
    kind, k, n = "q6_K", 1024, 640
    w32 = synth.normal(7400, (n, k), 0.02)
    blocks, fw = _framework_bytes(cr, kind, w32, n, k)
    x = synth.normal(7401, (1, k))
    fw.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    _run(["fc", kind, k, n, 1, 1, 0, 0, tmp_path / "w.bin", tmp_path / "x.bin", "-", tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(1, n)
    ref = cr.gemm(cr.oracle(), kind, x, blocks, n)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert int(got.argmax()) == int(ref.argmax())


def test_moe_incremental_forwarding(cr, tmp_path):
    t, h, i, e, k = 12, 512, 256, 8, 2
    gate, up, down = [], [], []
    for x in range(e):
        gate.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(7500 + 3 * x, (i, h), 0.02)))
        up.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(7501 + 3 * x, (i, h), 0.02)))
        down.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(7502 + 3 * x, (h, i), 0.02)))
    xin = synth.normal(7600, (t, h))
    wr = synth.normal(7601, (h, e), 0.1)
    logits = (xin.astype(np.float64) @ wr.astype(np.float64)).astype(np.float32)
    ref_y, _, _ = cr.moe_forward(xin, logits, gate, up, down, k)
    # the layer's tensors: router [H x E] fp32, then up_e, gate_e, down_e in x8 layout
    wr.tofile(tmp_path / "router.bin")
    with open(tmp_path / "experts.bin", "wb") as f:
        for x in range(e):
            f.write(cr.repack_x8(cr.oracle(), "q4_K", up[x], i, h).tobytes())
            f.write(cr.repack_x8(cr.oracle(), "q4_K", gate[x], i, h).tobytes())
            f.write(cr.repack_x8(cr.oracle(), "q4_K", down[x], h, i).tobytes())
    xin.tofile(tmp_path / "x.bin")
    _run(["moe", "q4_K", t, h, i, e, k, 1, tmp_path / "router.bin", tmp_path / "experts.bin",
          tmp_path / "x.bin", tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(t, h)
    err = np.abs(got - ref_y).max() / np.abs(ref_y).max()
    assert err <= 2e-4, err  # router logits computed on the device differ in the last bits


@pytest.mark.parametrize("how", ["read", "poke"])
def test_fc_sees_weights_rewritten_in_place(cr, tmp_path, how):
    """A weight tensor whose bytes change after a first forward -- read again from a model
    file through Layer::read, or rewritten behind the layer's back -- must not be served
    from the device copy of its old content."""
    kind, k, n, height = "q4_K", 512, 384, 3
    blocks_a, fw_a = _framework_bytes(cr, kind, synth.normal(7700, (n, k), 0.02), n, k)
    blocks_b, fw_b = _framework_bytes(cr, kind, synth.normal(7701, (n, k), 0.02), n, k)
    x = synth.normal(7702, (height, k))
    fw_a.tofile(tmp_path / "wa.bin")
    fw_b.tofile(tmp_path / "wb.bin")
    x.tofile(tmp_path / "x.bin")
    _run(["fcreload", kind, k, n, height, tmp_path / "wa.bin", tmp_path / "wb.bin", tmp_path / "x.bin", how,
          tmp_path / "ya.bin", tmp_path / "yb.bin"])
    for name, blocks in (("ya.bin", blocks_a), ("yb.bin", blocks_b)):
        got = np.fromfile(tmp_path / name, np.float32).reshape(height, n)
        ref = cr.gemm(cr.oracle(), kind, x, blocks, n)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), name


def test_moe_forwarding_keeps_softmax_values(cr, tmp_path):
    """MoELayer::forwarding (qwen_moe_layer.cpp:161-259) weights the experts with the softmax
    values as they are, without dividing by their sum."""
    t, h, i, e, k = 6, 256, 256, 8, 2
    q = lambda s, shape: cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(s, shape, 0.02))
    gate = [q(7800 + 3 * x, (i, h)) for x in range(e)]
    up = [q(7801 + 3 * x, (i, h)) for x in range(e)]
    down = [q(7802 + 3 * x, (h, i)) for x in range(e)]
    xin = synth.normal(7900, (t, h))
    wr = synth.normal(7901, (h, e), 0.1)
    logits = (xin.astype(np.float64) @ wr.astype(np.float64)).astype(np.float32)
    ref_y, _, ref_w = cr.moe_forward(xin, logits, gate, up, down, k, renormalize=False)
    assert (ref_w.sum(1) < 0.99).all()
    wr.tofile(tmp_path / "router.bin")
    with open(tmp_path / "experts.bin", "wb") as f:
        for x in range(e):
            f.write(cr.repack_x8(cr.oracle(), "q4_K", up[x], i, h).tobytes())
            f.write(cr.repack_x8(cr.oracle(), "q4_K", gate[x], i, h).tobytes())
            f.write(cr.repack_x8(cr.oracle(), "q4_K", down[x], h, i).tobytes())
    xin.tofile(tmp_path / "x.bin")
    _run(["moe", "q4_K", t, h, i, e, k, 0, tmp_path / "router.bin", tmp_path / "experts.bin",
          tmp_path / "x.bin", tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(t, h)
    err = np.abs(got - ref_y).max() / np.abs(ref_y).max()
    assert err <= 2e-4, err  # router logits computed on the device differ in the last bits
