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


@pytest.mark.parametrize("kind,k,n", [("q4_K", 1024, 1056), ("q4_K", 512, 256), ("q6_K", 512, 384), ("q4_0", 512, 320)])
def test_fc_decode_step_of_a_batch_is_one_call_with_each_entry_s_bits(cr, tmp_path, kind, k, n):
    """A decode step (to - from == 1) of a batch of eight: the layer sends the eight rows as one
    hipq_matmul_each_row call; every entry carries the bits of the M = 1 product the reference
    computes for it (fc_layer.cpp:266-296), with the reference's offset rule for the input, and
    the rest of the output is left alone."""
    batch, height = 8, 4
    w32 = synth.normal(7350, (n, k), 0.02)
    blocks, fw = _framework_bytes(cr, kind, w32, n, k)
    x = synth.normal(7351, (batch, height, k))
    x.reshape(-1)[1 * height * n + 3] = 6.5   # entry 1: +amax before -amax (the quantizers' sign rules)
    x.reshape(-1)[1 * height * n + 9] = -6.5
    fw.tofile(tmp_path / "w.bin")
    x.tofile(tmp_path / "x.bin")
    if (batch - 1) * height * n + k > x.size:
        pytest.skip("the reference's offset rule leaves the input tensor")
    _run(["fc", kind, k, n, batch, height, 3, 4, tmp_path / "w.bin", tmp_path / "x.bin", "-", tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, height, n)
    for b in range(batch):
        xin = x.reshape(-1)[b * height * n:][:k].reshape(1, k)
        ref = cr.gemm(cr.oracle(), kind, xin, blocks, n)
        assert np.array_equal(got[b, :1].view(np.uint32), ref.view(np.uint32)), (kind, b)
        assert np.all(got[b, 1:] == -12345.0)


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
    logits = cr.router_logits(xin, wr, k)
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
    assert err <= TOL, err  # router logits computed on the device differ in the last bits only


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
    logits = cr.router_logits(xin, wr, k)
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
    assert err <= TOL, err  # router logits computed on the device differ in the last bits only


@pytest.mark.parametrize("kind,k,nq,nk,nv,height,frm,to", [
    ("q4_0", 1024, 2048, 1024, 1024, 1, 7, 8),    # a decode step of the Qwen3-0.6B shape: one launch
    ("q4_K", 1024, 512, 256, 256, 1, 0, 1),
    ("q6_K", 512, 256, 256, 128, 1, 3, 4),
    ("q4_0", 1024, 512, 256, 256, 24, 0, 17),    # prefill: rows [0, 17) of 24
])
def test_qkv_layer_matches_oracle_bit_for_bit(cr, tmp_path, kind, k, nq, nk, nv, height, frm, to):
    """qkv_layer created through the context: three quantized products of one activation
    (qkv_layer.cpp:132-181). Decode rows and Q4_0 prefill rows follow the reference's evaluation
    order, so the outputs carry the oracle's bits."""
    ws, fws = [], []
    for j, n in enumerate((nq, nk, nv)):
        blocks, fw = _framework_bytes(cr, kind, synth.normal(8000 + j, (n, k), 0.02), n, k)
        ws.append(blocks)
        fws.append(fw)
    x = synth.normal(8010 + height, (height, k))
    with open(tmp_path / "w.bin", "wb") as f:
        for fw in fws:
            f.write(fw.tobytes())
    x.tofile(tmp_path / "x.bin")
    out = _run(["qkv", kind, k, nq, nk, nv, height, frm, to, tmp_path / "w.bin", tmp_path / "x.bin",
                tmp_path / "y.bin"])
    assert "QKV DONE" in out
    got = np.fromfile(tmp_path / "y.bin", np.float32)
    rows, off = to - frm, 0
    for blocks, n in zip(ws, (nq, nk, nv)):
        y = got[off:off + height * n].reshape(height, n)
        off += height * n
        ref = cr.gemm(cr.oracle(), kind, x[:rows], blocks, n)
        assert np.array_equal(y[:rows].view(np.uint32), ref.view(np.uint32))
        assert np.all(y[rows:] == -12345.0)


@pytest.mark.parametrize("batch,height,frm,to", [(1, 1, 11, 12), (1, 9, 0, 9), (2, 6, 0, 4)])
def test_tied_lm_head_matches_oracle(cr, tmp_path, batch, height, frm, to):
    """tie_word_embeddings with `unit`: hidden = input . table^T for one row per batch entry, row 0
    of a one-token step, else the step's last row (tie_word_embedding.cpp:252-303); the table is
    the Q6_K embedding matrix, unit rows of K values."""
    kind, k, unit = "q6_K", 512, 1000
    table = cr.quantize_weights(cr.oracle(), kind, synth.normal(8100, (unit, k), 0.02))
    x = synth.normal(8101 + height, (batch, height, k))
    table.tofile(tmp_path / "t.bin")
    x.tofile(tmp_path / "x.bin")
    _run(["lmhead", kind, k, unit, batch, height, frm, to, tmp_path / "t.bin", tmp_path / "x.bin",
          tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, height, unit)
    row = 0 if to - frm == 1 else to - 1
    for b in range(batch):
        ref = cr.gemm(cr.oracle(), kind, x[b, row:row + 1], table, unit)
        assert np.array_equal(got[b, row].view(np.uint32), ref[0].view(np.uint32))
        rest = np.delete(got[b], row, axis=0)
        assert np.all(rest == -12345.0)


@pytest.mark.parametrize("kind", ["q6_K", "fp32"])
def test_tied_embedding_rows(cr, tmp_path, kind):
    """tie_word_embeddings without `unit`: row `id` of the table per input id, dequantized for
    Q6_K (tie_word_embedding.cpp:183-250). Host work; here because the same layer object type
    serves both ends of the model."""
    in_dim, out_dim, batch, width = 300, 512, 2, 5
    w32 = synth.normal(8200, (in_dim, out_dim), 0.02)
    if kind == "q6_K":
        table = cr.quantize_weights(cr.oracle(), kind, w32)
        rows = cr.dequantize(cr.oracle(), kind, table, in_dim * out_dim).reshape(in_dim, out_dim)
    else:
        table, rows = w32, w32
    ids = np.array([[0, 299, 17, 5, 17], [1, 2, 3, 4, 250]], np.float32)
    table.tofile(tmp_path / "t.bin")
    ids.tofile(tmp_path / "i.bin")
    _run(["embed", kind, in_dim, out_dim, batch, width, 0, 3, tmp_path / "t.bin", tmp_path / "i.bin",
          tmp_path / "y.bin"])
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, width, out_dim)
    for b in range(batch):
        for i in range(3):
            assert np.array_equal(got[b, i].view(np.uint32), rows[int(ids[b, i])].view(np.uint32))
        assert np.all(got[b, 3:] == -12345.0)


def _moe_file(cr, path, kind, e, i, h, wr, experts, gate_bias=None, biases=None):
    """every weight of an MoE layer in the order it requests them"""
    gate, up, down = experts
    with open(path, "wb") as f:
        f.write(wr.tobytes())
        if gate_bias is not None:
            f.write(gate_bias.tobytes())
        for x in range(e):
            f.write(cr.repack_x8(cr.oracle(), kind, up[x], i, h).tobytes())
            if biases:
                f.write(biases[1][x].tobytes())
            f.write(cr.repack_x8(cr.oracle(), kind, gate[x], i, h).tobytes())
            if biases:
                f.write(biases[0][x].tobytes())
            f.write(cr.repack_x8(cr.oracle(), kind, down[x], h, i).tobytes())
            if biases:
                f.write(biases[2][x].tobytes())


def _moe_case(cr, seed, t, h, i, e, k):
    q = lambda s, shape: cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(s, shape, 0.02))
    experts = ([q(seed + 3 * x, (i, h)) for x in range(e)], [q(seed + 3 * x + 1, (i, h)) for x in range(e)],
               [q(seed + 3 * x + 2, (h, i)) for x in range(e)])
    xin = synth.normal(seed + 100, (t, h))
    wr = synth.normal(seed + 101, (h, e), 0.1)
    logits = cr.router_logits(xin, wr, k)
    return experts, xin, wr, logits


def test_cached_moe_layer(cr, tmp_path):
    """moe_cached_slim (qwen_moe_layer_cached.cpp:266-470): virtual expert tensors, loaded through
    Layer::read, activated once, kept in HBM and left deactivated. Checked against the oracle of
    the cached layer's own arithmetic (one product per expert over its tokens, the x86 swiglu for
    more than one token, orc_moe_forward_cached): every pair here carries its M = 1 bits instead,
    which is inside the fp32 tolerance of that."""
    t, h, i, e, k = 12, 512, 256, 8, 2
    experts, xin, wr, logits = _moe_case(cr, 8300, t, h, i, e, k)
    ref_y, ref_idx, _ = cr.moe_forward_cached(xin, logits, *experts, k)
    counts = np.bincount(ref_idx.ravel(), minlength=e)
    assert (counts >= 4).any() and (counts % 4 != 0).any(), "both row rules of the batched products occur"
    _moe_file(cr, tmp_path / "w.bin", "q4_K", e, i, h, wr, experts)
    xin.tofile(tmp_path / "x.bin")
    out = _run(["moex", "moe_cached_slim", "q4_K", t, h, i, e, k, 1, tmp_path / "w.bin", tmp_path / "x.bin",
                tmp_path / "y.bin"])
    assert "active_virtual=0" in out
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(t, h)
    assert np.abs(got - ref_y).max() / np.abs(ref_y).max() <= TOL
    # forwarding() of the cached layer is a no-op, as in the reference
    _run(["moex", "moe_cached_slim", "q4_K", t, h, i, e, k, 0, tmp_path / "w.bin", tmp_path / "x.bin",
          tmp_path / "y0.bin"])
    assert np.all(np.fromfile(tmp_path / "y0.bin", np.float32) == -12345.0)


@pytest.mark.parametrize("layer,incremental", [("gpt_oss_moe", 1), ("gpt_oss_moe", 0),
                                               ("gpt_oss_moe_slim_cached", 1)])
def test_gpt_oss_moe_layers(cr, tmp_path, layer, incremental):
    """gpt_oss_moe and its cached twin through the context. The router bias enters only in the
    uncached layer's incremental_forwarding (gpt_oss_moe_layer.cpp:500-504; not :209-212, not
    gpt_oss_moe_layer_cached.cpp:243-246), and forwarding() keeps the softmax values as they are."""
    t, h, i, e, k = 9, 256, 256, 8, 2
    experts, xin, wr, logits = _moe_case(cr, 8400, t, h, i, e, k)
    cached = layer == "gpt_oss_moe_slim_cached"
    rb = synth.normal(8450, (e,), 2.0)
    # biases wide enough that biased gate and up values pass the cached layer's limit of 7
    gb = synth.normal(8451, (e, i), 3.0)
    ub = synth.normal(8452, (e, i), 3.0)
    db = synth.normal(8453, (e, h), 0.3)
    with_bias = layer == "gpt_oss_moe" and incremental == 1
    lg = cr.router_logits(xin, wr, k, rb) if with_bias else logits
    if cached:
        # the cached layer clamps (gpt_oss_moe_layer_cached.cpp:497-507); its oracle is the cached one
        ref_y, ref_idx, _ = cr.moe_forward_cached(xin, lg, *experts, k, "q4_K", True, gb, ub, db)
        unclamped, _, _ = cr.moe_forward_cached(xin, lg, *experts, k, "q4_K", True, gb, ub, db, limit=1e30)
        assert np.abs(unclamped - ref_y).max() > 1e-2 * np.abs(ref_y).max(), "the clamps must act in this case"
    else:
        ref_y, ref_idx, _ = cr.moe_forward_gpt_oss(xin, lg, *experts, gb, ub, db, k, renormalize=bool(incremental))
    _, other_idx, _ = cr.moe_forward_gpt_oss(xin, logits if with_bias else cr.router_logits(xin, wr, k, rb),
                                             *experts, gb, ub, db, k, renormalize=bool(incremental))
    assert not np.array_equal(ref_idx, other_idx), "the router bias must matter in this case"
    _moe_file(cr, tmp_path / "w.bin", "q4_K", e, i, h, wr, experts, gate_bias=rb, biases=(gb, ub, db))
    xin.tofile(tmp_path / "x.bin")
    out = _run(["moex", layer, "q4_K", t, h, i, e, k, incremental, tmp_path / "w.bin", tmp_path / "x.bin",
                tmp_path / "y.bin"])
    assert "active_virtual=0" in out
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(t, h)
    assert np.abs(got - ref_y).max() / np.abs(ref_y).max() <= TOL


@pytest.mark.parametrize("kind,k,n,batch,height,frm,to", [("q4_0", 1024, 3072, 1, 1, 5, 6),   # decode: one launch
                                                          ("q4_K", 1024, 768, 1, 20, 0, 0),    # forwarding
                                                          ("q4_0", 512, 256, 2, 8, 0, 5)])     # prefill step, batch 2
def test_mlp_swiglu_layer(cr, tmp_path, kind, k, n, batch, height, frm, to):
    """mlp_swiglu through the context: ffn_up, ffn_gate and the SwiGLU between them
    (causal_lm.cpp:672-695) as one layer; weights in the file order of the two FCs."""
    up, fup = _framework_bytes(cr, kind, synth.normal(8500, (n, k), 0.05), n, k)
    gate, fgate = _framework_bytes(cr, kind, synth.normal(8501, (n, k), 0.05), n, k)
    x = synth.normal(8502 + height, (batch, height, k))
    with open(tmp_path / "w.bin", "wb") as f:
        f.write(fup.tobytes())
        f.write(fgate.tobytes())
    x.tofile(tmp_path / "x.bin")
    out = _run(["mlp", kind, k, n, batch, height, frm, to, tmp_path / "w.bin", tmp_path / "x.bin", tmp_path / "y.bin"])
    assert "MLP DONE" in out
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, height, n)
    rows = height if to == 0 else to - frm
    for b in range(batch):
        y = cr.gemm(cr.oracle(), kind, x[b, :rows], up, n)
        z = cr.gemm(cr.oracle(), kind, x[b, :rows], gate, n)
        ref = cr.swiglu(y, z)
        assert np.abs(got[b, :rows] - ref).max() / np.abs(ref).max() <= TOL
        assert np.all(got[b, rows:] == -12345.0)


@pytest.mark.parametrize("kind,k,n,nd,batch,height,frm,to", [("q4_0", 1024, 3072, 1024, 1, 1, 5, 6),   # decode row
                                                             ("q4_K", 1024, 768, 1024, 1, 20, 0, 0),    # forwarding
                                                             ("q4_0", 512, 256, 512, 2, 8, 0, 5)])      # prefill step
def test_mlp_swiglu_layer_with_the_down_projection(cr, tmp_path, kind, k, n, nd, batch, height, frm, to):
    """mlp_swiglu with down_unit: the four layers of CausalLM::createMlp (causal_lm.cpp:671-705) as one, the
    hidden rows never on the host; weights in the file order of the three FCs."""
    up, fup = _framework_bytes(cr, kind, synth.normal(8600, (n, k), 0.05), n, k)
    gate, fgate = _framework_bytes(cr, kind, synth.normal(8601, (n, k), 0.05), n, k)
    down, fdown = _framework_bytes(cr, kind, synth.normal(8602, (nd, n), 0.05), nd, n)
    x = synth.normal(8603 + height, (batch, height, k))
    with open(tmp_path / "w.bin", "wb") as f:
        f.write(fup.tobytes())
        f.write(fgate.tobytes())
        f.write(fdown.tobytes())
    x.tofile(tmp_path / "x.bin")
    out = _run(["mlp", kind, k, n, batch, height, frm, to, tmp_path / "w.bin", tmp_path / "x.bin", tmp_path / "y.bin",
                nd])
    assert "MLP DONE" in out
    got = np.fromfile(tmp_path / "y.bin", np.float32).reshape(batch, height, nd)
    rows = height if to == 0 else to - frm
    for b in range(batch):
        hidden = cr.swiglu(cr.gemm(cr.oracle(), kind, x[b, :rows], up, n), cr.gemm(cr.oracle(), kind, x[b, :rows], gate, n))
        ref = cr.gemm(cr.oracle(), kind, hidden, down, nd)
        assert np.abs(got[b, :rows] - ref).max() / np.abs(ref).max() <= TOL
        assert np.all(got[b, rows:] == -12345.0)


def test_moe_sees_expert_weights_rewritten_in_place(cr, tmp_path):
    """The MoE layer remembers its experts' device handles between calls; experts whose bytes change at the
    same addresses (a second model read into the same tensors) must be uploaded again."""
    t, h, i, e, k = 6, 512, 256, 8, 2
    sets = []
    for base in (7900, 7950):
        gate = [cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(base + 3 * x, (i, h), 0.02)) for x in range(e)]
        up = [cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(base + 3 * x + 1, (i, h), 0.02)) for x in range(e)]
        down = [cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(base + 3 * x + 2, (h, i), 0.02)) for x in range(e)]
        sets.append((gate, up, down))
    xin = synth.normal(7990, (t, h))
    wr = synth.normal(7991, (h, e), 0.1)
    logits = cr.router_logits(xin, wr, k)
    wr.tofile(tmp_path / "router.bin")
    for name, (gate, up, down) in zip(("a.bin", "b.bin"), sets):
        with open(tmp_path / name, "wb") as f:
            for x in range(e):
                f.write(cr.repack_x8(cr.oracle(), "q4_K", up[x], i, h).tobytes())
                f.write(cr.repack_x8(cr.oracle(), "q4_K", gate[x], i, h).tobytes())
                f.write(cr.repack_x8(cr.oracle(), "q4_K", down[x], h, i).tobytes())
    xin.tofile(tmp_path / "x.bin")
    _run(["moe", "q4_K", t, h, i, e, k, 1, tmp_path / "router.bin", tmp_path / "a.bin", tmp_path / "x.bin",
          tmp_path / "ya.bin", tmp_path / "b.bin", tmp_path / "yb.bin"])
    for name, (gate, up, down) in zip(("ya.bin", "yb.bin"), sets):
        ref_y, _, _ = cr.moe_forward(xin, logits, gate, up, down, k)
        got = np.fromfile(tmp_path / name, np.float32).reshape(t, h)
        assert np.abs(got - ref_y).max() / np.abs(ref_y).max() <= TOL, name
