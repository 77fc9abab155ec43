"""CPU: pin the oracle (oracle/nntr_oracle.c).

Three kinds of evidence, none of which retypes the oracle's own formulas:
 1. bit-for-bit equality with the reference library built from the reference's own
    sources (oracle/_ref), when that library is present;
 2. closed forms the block formats fix: matmul == dot(dequant(W), dequant(QA)) in
    double; repack is an invertible byte permutation; quantizer invariants;
 3. committed golden digests of oracle outputs on seeded inputs (tests/golden),
    produced where the reference library was available, so drift of the oracle is
    caught on machines without it.
"""
import json
import os

import numpy as np
import pytest

import cpuref as cr
from nntrainer_amd import synth

KINDS = ["q4_0", "q4_K", "q6_K"]
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "oracle_digests.json")
needs_ref = pytest.mark.skipif(cr.ref() is None, reason="reference library not built here")


def _w(seed, n, k, sigma=0.02):
    w = synth.normal(seed, (n, k), sigma)
    w[1, :256] = 0.0       # all-zero super-block / blocks
    w[2, 256:288] = 0.0    # one zero sub-block
    w[3, 0:32] = 0.01      # constant sub-block (max == min)
    return w


# ------------------------------------------------------------------ 1. vs reference
@needs_ref
def test_fp16_conversions_match_reference():
    o, r = cr.oracle(), cr.ref()
    for h in range(0, 65536, 1):
        a, b = o.orc_fp16_to_fp32(h), r.ref_fp16_to_fp32(h)
        assert np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32) or (a != a and b != b)
    rng = np.random.default_rng(0)
    fs = np.concatenate([rng.standard_normal(20000).astype(np.float32) * s
                         for s in (1, 1e-3, 1e-5, 1e-7, 300, 7e4)])
    edge = np.array([65504, 65519.99, 65520, 65536, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 0, -0.0,
                     np.inf, -np.inf, 6.1e-5, 6.0975e-5], np.float32)
    for f in np.concatenate([fs, edge]):
        assert o.orc_fp32_to_fp16(float(f)) == r.ref_fp32_to_fp16(float(f)), f


@needs_ref
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("sigma", [0.02, 1.0])
def test_weight_quantizer_bytes_match_reference(kind, sigma):
    """4.2 million weights per format and scale (16 384 super-blocks of 256): the searches
    are order-sensitive fp32 code and every configuration's weights come out of them."""
    w = _w(3, 1024, 4096, sigma)
    assert np.array_equal(cr.quantize_weights(cr.oracle(), kind, w), cr.quantize_weights(cr.ref(), kind, w))


@needs_ref
@pytest.mark.parametrize("kind", KINDS)
def test_weight_quantizer_bytes_match_reference_uniform(kind):
    """The inputs of the reference's own quantizer tests: uniform in (-1, 1)
    (unittest_nntrainer_cpu_backend.cpp:35-48), plus rows with exact zeros and ties."""
    u = np.random.default_rng(9).uniform(-1.0, 1.0, (512, 2048)).astype(np.float32)
    u[0, :256] = 0.0
    u[1, :64] = 0.25
    u[2, ::2] = -u[2, 1::2]
    assert np.array_equal(cr.quantize_weights(cr.oracle(), kind, u), cr.quantize_weights(cr.ref(), kind, u))


@needs_ref
@pytest.mark.parametrize("kind", KINDS)
def test_dequantize_matches_reference(kind):
    q = cr.quantize_weights(cr.ref(), kind, _w(4, 64, 1024))
    a, b = cr.dequantize(cr.oracle(), kind, q, 64 * 1024), cr.dequantize(cr.ref(), kind, q, 64 * 1024)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@needs_ref
@pytest.mark.parametrize("kind", ["q4_0", "q4_K"])
def test_repack_matches_reference(kind):
    q = cr.quantize_weights(cr.ref(), kind, _w(5, 64, 1024))
    assert np.array_equal(cr.repack_x8(cr.oracle(), kind, q, 64, 1024), cr.repack_x8(cr.ref(), kind, q, 64, 1024))


def _act_cases(k):
    x = synth.normal(11, (16, k))
    x[0, :] = 0.0
    x[2, 5] = 9.5; x[2, 9] = -9.5
    x[3, 5] = -9.5; x[3, 9] = 9.5
    x[4, :] *= 1e-6
    x[5, :] *= 1e4
    return x


@needs_ref
@pytest.mark.parametrize("kind", ["q8_0", "q8_K"])
def test_activation_quantizers_match_reference(kind):
    x = _act_cases(1024)
    adv = np.load(os.path.join(os.path.dirname(__file__), "golden", "q8k_rounding_adversaries.npy"))
    x = np.concatenate([x, adv.reshape(-1, 256)[:24].reshape(-1, 1024)])
    x = x[: (len(x) // 4) * 4]
    o, r = cr.oracle(), cr.ref()
    assert np.array_equal(cr.quantize_act(o, kind, x, "row"), cr.quantize_act(r, kind, x, "row"))
    mo = cr.quantize_act(o, kind, x, "mat")
    inter = np.stack([cr.interleave4(kind, mo[4 * g:4 * g + 4], 1024) for g in range(len(x) // 4)])
    assert np.array_equal(inter, cr.quantize_act(r, kind, x, "mat"))


@needs_ref
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m", [1, 3, 4, 7, 16, 35])
def test_matmul_bits_match_reference(kind, m):
    """Same bits as the reference wrapper, for GEMV (M=1), the 4-row GEMM path and the
    leftover-row path (M % 4 != 0)."""
    n, k = 128, 1024
    q = cr.quantize_weights(cr.ref(), kind, _w(6, n, k))
    a = synth.normal(60 + m, (m, k))
    co, cc = cr.gemm(cr.oracle(), kind, a, q, n), cr.gemm(cr.ref(), kind, a, q, n)
    assert np.array_equal(co.view(np.uint32), cc.view(np.uint32))


# ------------------------------------------------------------------ 2. closed forms
@pytest.mark.parametrize("kind", KINDS)
def test_matmul_equals_dequantized_dot(kind):
    """C == dequant(QA) . dequant(W)^T evaluated in double (a textbook dot product):
    catches a wrong nibble order, scale index, sign or a dropped min term."""
    n, k, m = 96, 1024, 5
    o = cr.oracle()
    q = cr.quantize_weights(o, kind, _w(7, n, k))
    a = synth.normal(70, (m, k))
    wd = cr.dequantize(o, kind, q, n * k).reshape(n, k).astype(np.float64)
    if kind == "q4_0":
        qa = cr.quantize_act(o, "q8_0", a)
        ad = np.stack([cr.dequantize(o, "q8_0", qa[i], k) for i in range(m)]).astype(np.float64)
    else:
        var = ["mat" if (kind == "q4_K" and i < (m // 4) * 4) else "row" for i in range(m)]
        ad = np.stack([cr.dequantize(o, "q8_K", cr.quantize_act(o, "q8_K", a[i:i + 1], var[i])[0], k)
                       for i in range(m)]).astype(np.float64)
    want = ad @ wd.T
    got = cr.gemm(o, kind, a, q, n)
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-6


@pytest.mark.parametrize("kind", KINDS)
def test_weight_quantizer_round_trip_error(kind):
    """Quantize -> dequantize error stays within the format's step (the reference's own
    acceptance is an mse bound, unittest_nntrainer_cpu_backend.cpp:182-293)."""
    o = cr.oracle()
    w = synth.normal(8, (64, 1024), 0.02)
    back = cr.dequantize(o, kind, cr.quantize_weights(o, kind, w), w.size).reshape(w.shape)
    rel = np.abs(back - w).max() / np.abs(w).max()
    assert rel < {"q4_0": 0.09, "q4_K": 0.07, "q6_K": 0.02}[kind]
    mse = float(((back - w) ** 2).mean())
    assert mse < 1e-5


@pytest.mark.parametrize("kind", ["q4_0", "q4_K"])
def test_repack_is_an_invertible_permutation(kind):
    o = cr.oracle()
    q = cr.quantize_weights(o, kind, _w(9, 64, 1024))
    x8 = cr.repack_x8(o, kind, q, 64, 1024)
    assert x8.size == q.size and not np.array_equal(x8, q)
    assert np.array_equal(cr.unpack_x8(kind, x8, 64, 1024), q)
    # repack refuses row counts that are not multiples of 8 (reference returns -1)
    out = np.zeros(18 * 12 * 2, np.uint8)
    assert o.orc_repack_q4_0_x8(out.ctypes.data, out.ctypes.data, 12, 64) == -1


def test_activation_quantizer_invariants():
    o = cr.oracle()
    x = _act_cases(1024)
    for variant in ("row", "mat"):
        blk = cr.quantize_act(o, "q8_K", x, variant).reshape(len(x), -1, 292)
        d = blk[..., :4].copy().view(np.float32)[..., 0]
        qs = blk[..., 4:260].copy().view(np.int8).astype(np.int32)
        bs = blk[..., 260:].copy().view(np.int16).astype(np.int32)
        assert (np.abs(qs) <= 127).all() or variant == "mat"
        assert np.array_equal(qs.reshape(len(x), -1, 16, 16).sum(-1), bs)       # group sums consistent
        xb = x.reshape(len(x), -1, 256)
        assert (np.abs(d[..., None] * qs - xb) <= np.abs(d[..., None]) * 0.5000001 + 1e-30).all()
        assert (d[0] == 0).all() and (qs[0] == 0).all()                         # all-zero row
    # sign rule when +amax and -amax both occur: row follows the first, mat a positive hit
    r2 = cr.quantize_act(o, "q8_K", x[2:4], "row").reshape(2, -1, 292)[:, 0, :4].copy().view(np.float32)
    m2 = cr.quantize_act(o, "q8_K", x[2:4], "mat").reshape(2, -1, 292)[:, 0, :4].copy().view(np.float32)
    assert r2[0, 0] < 0 and r2[1, 0] > 0 and m2[0, 0] < 0 and m2[1, 0] < 0
    b0 = cr.quantize_act(o, "q8_0", x).reshape(len(x), -1, 34)
    q0 = b0[..., 2:].copy().view(np.int8)
    assert (np.abs(q0.astype(np.int32)) <= 127).all()
    assert (np.abs(q0).max(-1)[1] == 127).all()  # the max element maps to +-127


def test_moe_equals_dense_per_token_evaluation():
    """MoE block == for every token, softmax over its top-k logits as weights of the
    SwiGLU MLPs of those experts, each built from the oracle's single-row matmul."""
    o = cr.oracle()
    t, h, i, e, k = 6, 256, 256, 8, 3
    gate = [cr.quantize_weights(o, "q4_K", synth.normal(100 + 3 * x, (i, h), 0.02)) for x in range(e)]
    up = [cr.quantize_weights(o, "q4_K", synth.normal(101 + 3 * x, (i, h), 0.02)) for x in range(e)]
    down = [cr.quantize_weights(o, "q4_K", synth.normal(102 + 3 * x, (h, i), 0.02)) for x in range(e)]
    x = synth.normal(200, (t, h))
    logits = synth.normal(201, (t, e))
    y, idx, wt = cr.moe_forward(x, logits, gate, up, down, k)
    f32 = np.float32
    want = np.zeros((t, h), np.float64)
    for tt in range(t):
        order = np.argsort(-logits[tt], kind="stable")[:k]
        assert set(order) == set(idx[tt])
        lw = np.exp(logits[tt, order].astype(np.float64) - logits[tt, order].max())
        lw /= lw.sum()  # renormalised softmax == softmax over the selected logits
        for ee, ww in zip(order, lw):
            g = cr.gemm(o, "q4_K", x[tt:tt + 1], gate[ee], i)[0]
            u = cr.gemm(o, "q4_K", x[tt:tt + 1], up[ee], i)[0]
            # acti_func.h:286-288, 400-405 taken literally: sigmoid = (float)(1.0 / (1.0 + exp(-x)))
            # with exp returning float, then two fp32 multiplies
            en = np.exp(-g.astype(np.float64)).astype(f32)
            sig = (1.0 / (1.0 + en.astype(np.float64))).astype(f32)
            hh = (sig * g).astype(f32) * u
            want[tt] += ww * cr.gemm(o, "q4_K", hh[None], down[ee], h)[0].astype(np.float64)
    assert np.abs(y - want).max() / np.abs(want).max() < 1e-5
    assert np.abs(wt.sum(1) - 1).max() < 1e-6
    # the forwarding path (qwen_moe_layer.cpp:161-259) keeps the softmax values as they are
    y0, idx0, wt0 = cr.moe_forward(x, logits, gate, up, down, k, renormalize=False)
    assert np.array_equal(idx0, idx)
    full = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
    full /= full.sum(1, keepdims=True)
    assert np.abs(wt0 - np.take_along_axis(full, idx0.astype(np.int64), 1)).max() < 1e-6
    scale = wt0.astype(np.float64).sum(1, keepdims=True)  # y0 = y * (sum of the kept softmax values)
    assert np.abs(y0 - want * scale).max() / np.abs(want).max() < 1e-5


def test_gpt_oss_moe_reduces_to_known_cases():
    """The GPT-OSS block of the oracle (gpt_oss_moe_layer.cpp:372-449), pinned three ways.
    (1) With up_bias = -1, the other biases 0 and alpha = 1 its activation is silu(g) * u: the
    block must then equal the Qwen block, whose own pins are above (float against double
    exponential: 1e-6). (2) alpha = 0 makes the sigmoid 1/2 whatever g is: h = g/2 * (u + 1),
    evaluated here from the oracle's single-row products with nonzero biases; a dropped bias, a
    missing + 1 or a bias on the wrong side of the activation fails it. (3) The down bias enters
    after the product and before the routing weight: y(db) - y(0) = sum_k w_k db[e_k]."""
    o = cr.oracle()
    t, h, i, e, k = 5, 256, 256, 6, 2
    gate = [cr.quantize_weights(o, "q4_K", synth.normal(300 + 3 * x, (i, h), 0.02)) for x in range(e)]
    up = [cr.quantize_weights(o, "q4_K", synth.normal(301 + 3 * x, (i, h), 0.02)) for x in range(e)]
    down = [cr.quantize_weights(o, "q4_K", synth.normal(302 + 3 * x, (h, i), 0.02)) for x in range(e)]
    x = synth.normal(400, (t, h))
    logits = synth.normal(401, (t, e))
    zi, zh = np.zeros((e, i), np.float32), np.zeros((e, h), np.float32)
    # (1)
    y_q, idx_q, wt_q = cr.moe_forward(x, logits, gate, up, down, k)
    y1, idx1, wt1 = cr.moe_forward_gpt_oss(x, logits, gate, up, down, zi, zi - 1, zh, k, alpha=1.0)
    assert np.array_equal(idx1, idx_q) and np.array_equal(wt1, wt_q)
    assert np.abs(y1 - y_q).max() / np.abs(y_q).max() < 1e-6
    # (2)
    gb, ub, db = synth.normal(402, (e, i), 0.3), synth.normal(403, (e, i), 0.3), synth.normal(404, (e, h), 0.3)
    y2, idx2, wt2 = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k, alpha=0.0)
    want = np.zeros((t, h), np.float64)
    for tt in range(t):
        for ee, ww in sorted(zip(idx2[tt], wt2[tt])):
            g = cr.gemm(o, "q4_K", x[tt:tt + 1], gate[ee], i)[0] + gb[ee]
            u = cr.gemm(o, "q4_K", x[tt:tt + 1], up[ee], i)[0] + ub[ee]
            hh = ((g / np.float32(2)) * (u + np.float32(1))).astype(np.float32)
            want[tt] += np.float64(ww) * (cr.gemm(o, "q4_K", hh[None], down[ee], h)[0].astype(np.float64) + db[ee])
    assert np.abs(y2 - want).max() / np.abs(want).max() < 1e-5
    # (3)
    ya, idx3, wt3 = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k)
    yb, _, _ = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, zh, k)
    shift = np.einsum("tk,tkh->th", wt3.astype(np.float64), db[idx3.astype(np.int64)].astype(np.float64))
    assert np.abs((ya.astype(np.float64) - yb) - shift).max() < 2e-5
    # and alpha is the sigmoid's slope: the default differs from alpha = 1 at this size
    yc, _, _ = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k, alpha=1.0)
    assert np.abs(ya - yc).max() / np.abs(ya).max() > 1e-2


def _swiglu_inputs():
    rng = np.random.default_rng(12)
    y = np.concatenate([rng.normal(0, s, 4099).astype(np.float32) for s in (0.05, 1, 6, 40)]
                       + [np.array([0, -0.0, 87.0, -87.0, 88.5, -88.5, 200, -200, 1e-39, -1e-39, 3e-38], np.float32)])
    z = rng.normal(0, 2, y.size).astype(np.float32)
    return y, z


@needs_ref
@pytest.mark.parametrize("alpha", [None, 1.702, 1.0])
def test_x86_swiglu_bits_match_reference(alpha):
    """orc_swiglu_x86 / orc_swiglu_alpha_x86 against avx2::swiglu of the reference build, bit for
    bit: small, ordinary and saturating arguments, denormals (read as zero while the routine
    runs), and lengths that end in the 8-wide and the masked step."""
    y, z = _swiglu_inputs()
    for n in (y.size, 16, 24, 29, 7, 1):
        a = cr.swiglu_x86(cr.oracle(), y[:n], z[:n], alpha)
        b = cr.swiglu_x86(cr.ref(), y[:n], z[:n], alpha)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), n


@needs_ref
def test_x86_swiglu_distance_from_the_expf_form():
    """How far the reference's x86 swiglu is from the expf form the C5 decoder's CPU leg and the
    dense-MLP oracle use: measured on gate values of the range a decoder produces (|y| up to 40),
    relative to the largest output. This number is what lets a 1e-4 test use either form."""
    y, z = _swiglu_inputs()
    keep = np.abs(y) < 60
    approx = cr.swiglu_x86(cr.ref(), y[keep], z[keep])
    exact = cr.swiglu(y[keep], z[keep])
    dist = np.abs(approx.astype(np.float64) - exact).max() / np.abs(exact).max()
    assert dist <= 2e-6, dist
    rel = np.abs(approx.astype(np.float64) - exact) / np.maximum(np.abs(exact), 1e-30)
    assert rel[np.abs(exact) > 1e-3].max() <= 1e-5


def _cached_moe_case(kind="q4_K", t=13, h=256, i=256, e=6, k=2, seed=500):
    o = cr.oracle()
    gate = [cr.quantize_weights(o, kind, synth.normal(seed + 3 * x, (i, h), 0.02)) for x in range(e)]
    up = [cr.quantize_weights(o, kind, synth.normal(seed + 1 + 3 * x, (i, h), 0.02)) for x in range(e)]
    down = [cr.quantize_weights(o, kind, synth.normal(seed + 2 + 3 * x, (h, i), 0.02)) for x in range(e)]
    x = synth.normal(seed + 100, (t, h))
    logits = synth.normal(seed + 101, (t, e))
    logits[0] = [9, 8, 0, 0, 0, 0][:e] if e >= 2 else logits[0]  # expert 0 and 1 certainly used
    return gate, up, down, x, logits


@needs_ref
@pytest.mark.parametrize("gpt_oss", [False, True])
def test_cached_moe_equals_composition_of_reference_routines(gpt_oss):
    """orc_moe_forward_cached against the cached layers' expert forward rebuilt here from the
    reference library's own routines: per expert one ref_gemm over its gathered tokens (its 4-row
    and leftover-row paths), ref_swiglu / the activation function by token count (Qwen) or the
    bias, ref_clamp, + 1 and ref_swiglu with alpha (GPT-OSS), one more ref_gemm, the routing weight,
    and the experts' [T x H] tensors added in ascending order. Bit for bit. Token counts per
    expert range over 1, 2..3 (leftover rows only), 4 and more (both paths)."""
    o, r = cr.oracle(), cr.ref()
    kind, t, h, i, e, k = "q4_K", 13, 256, 256, 6, 2
    gate, up, down, x, logits = _cached_moe_case(kind, t, h, i, e, k)
    logits[:, 5] = -30.0
    logits[3, 5] = 30.0  # expert 5 gets exactly one token
    gb, ub, db = synth.normal(601, (e, i), 3.0), synth.normal(602, (e, i), 3.0), synth.normal(603, (e, h), 0.3)
    y, idx, wt = cr.moe_forward_cached(x, logits, gate, up, down, k, kind, gpt_oss, gb, ub, db)
    counts = np.bincount(idx.ravel(), minlength=e)
    assert counts[5] == 1 and (counts >= 4).any() and ((counts > 1) & (counts % 4 != 0)).any()
    f32 = np.float32
    want = None
    import ctypes as c
    for ee in range(e):
        toks = [(tt, wt[tt, kk]) for tt in range(t) for kk in range(k) if idx[tt, kk] == ee]
        if not toks:
            continue
        tin = np.stack([x[tt] for tt, _ in toks])
        g = cr.gemm(r, kind, tin, gate[ee], i)
        u = cr.gemm(r, kind, tin, up[ee], i)
        if gpt_oss:
            g = (g + gb[ee]).astype(f32)
            u = (u + ub[ee]).astype(f32)
            gc, uc = np.empty_like(g), np.empty_like(u)
            r.ref_clamp(cr._ptr(g), cr._ptr(gc), c.c_size_t(g.size), c.c_float(np.finfo(f32).min), c.c_float(7.0))
            r.ref_clamp(cr._ptr(u), cr._ptr(uc), c.c_size_t(u.size), c.c_float(-7.0), c.c_float(7.0))
            uc = (uc + f32(1)).astype(f32)
            hh = np.stack([cr.swiglu_x86(r, gc[j], uc[j], 1.702) for j in range(len(toks))])
        elif len(toks) == 1:
            en = np.exp(-g.astype(np.float64)).astype(f32)
            sig = (1.0 / (1.0 + en.astype(np.float64))).astype(f32)
            hh = ((sig * g).astype(f32) * u).astype(f32)
        else:
            hh = np.stack([cr.swiglu_x86(r, g[j], u[j]) for j in range(len(toks))])
        od = cr.gemm(r, kind, hh, down[ee], h)
        if gpt_oss:
            od = (od + db[ee]).astype(f32)
        eo = np.zeros((t, h), f32)
        for j, (tt, ww) in enumerate(toks):
            eo[tt] = eo[tt] + (od[j] * f32(ww)).astype(f32)
        want = eo if want is None else (want + eo).astype(f32)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    if gpt_oss:  # the clamps are live: pre-activations beyond the limit exist in this case
        g0 = cr.gemm(o, kind, x, gate[0], i) + gb[0]
        assert (g0 > 7).any() and (np.abs(cr.gemm(o, kind, x, up[0], i) + ub[0]) > 7).any()


def test_cached_moe_reduces_to_the_per_token_layer():
    """Without the reference library: with one token every expert sees one row, where the cached
    Qwen layer evaluates exactly what the per-token layer does (same products, the activation
    function's sigmoid): the two oracles must agree bit for bit. With more tokens they differ only
    by the 4-row products' fp32 order and the approximate exponential: 2e-5 of the largest output.
    For GPT-OSS with limits beyond every pre-activation the same holds against the unclamped block,
    and with limit = 7 on large biases the outputs must differ (the clamp acts)."""
    kind, t, h, i, e, k = "q4_K", 9, 256, 256, 6, 2
    gate, up, down, x, logits = _cached_moe_case(kind, t, h, i, e, k, seed=700)
    y1, idx1, wt1 = cr.moe_forward_cached(x[:1], logits[:1], gate, up, down, k, kind)
    y0, idx0, wt0 = cr.moe_forward(x[:1], logits[:1], gate, up, down, k, kind)
    assert np.array_equal(idx1, idx0) and np.array_equal(wt1, wt0)
    assert np.array_equal(y1.view(np.uint32), y0.view(np.uint32))
    y, idx, wt = cr.moe_forward_cached(x, logits, gate, up, down, k, kind)
    yp, idxp, wtp = cr.moe_forward(x, logits, gate, up, down, k, kind)
    assert np.array_equal(idx, idxp) and np.array_equal(wt, wtp)
    assert 0 < np.abs(y - yp).max() <= 2e-5 * np.abs(yp).max()
    gb, ub, db = synth.normal(801, (e, i), 0.3), synth.normal(802, (e, i), 0.3), synth.normal(803, (e, h), 0.3)
    yg, _, _ = cr.moe_forward_cached(x, logits, gate, up, down, k, kind, True, gb, ub, db, limit=1e30)
    yu, _, _ = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k)
    assert np.abs(yg - yu).max() <= 2e-5 * np.abs(yu).max()
    big = synth.normal(804, (e, i), 4.0)
    yc, _, _ = cr.moe_forward_cached(x, logits, gate, up, down, k, kind, True, big, big, db, limit=7.0)
    yn, _, _ = cr.moe_forward_cached(x, logits, gate, up, down, k, kind, True, big, big, db, limit=1e30)
    assert np.abs(yc - yn).max() > 1e-2 * np.abs(yn).max()


# ------------------------------------------------------------------ 3. golden digests
def _digest_cases():
    o = cr.oracle()
    out = {}
    for kind in KINDS:
        w = _w(20, 64, 1024)
        q = cr.quantize_weights(o, kind, w)
        out["wquant_" + kind] = synth.digest(q)
        for m in (1, 6):
            out["gemm_%s_m%d" % (kind, m)] = synth.digest(cr.gemm(o, kind, synth.normal(21 + m, (m, 1024)), q, 64))
    x = _act_cases(1024)
    out["q8_0"] = synth.digest(cr.quantize_act(o, "q8_0", x))
    out["q8_K_row"] = synth.digest(cr.quantize_act(o, "q8_K", x, "row"))
    out["q8_K_mat"] = synth.digest(cr.quantize_act(o, "q8_K", x, "mat"))
    out["input_w"] = synth.digest(_w(20, 64, 1024))
    ys, zs = _swiglu_inputs()
    out["swiglu_x86"] = synth.digest(cr.swiglu_x86(o, ys, zs))
    out["swiglu_alpha_x86"] = synth.digest(cr.swiglu_x86(o, ys, zs, 1.702))
    gate, up, down, x, logits = _cached_moe_case()
    e, i, h = len(gate), 256, 256
    out["moe_cached_qwen"] = synth.digest(cr.moe_forward_cached(x, logits, gate, up, down, 2)[0])
    gb, ub, db = synth.normal(601, (e, i), 3.0), synth.normal(602, (e, i), 3.0), synth.normal(603, (e, h), 0.3)
    out["moe_cached_gpt_oss"] = synth.digest(cr.moe_forward_cached(x, logits, gate, up, down, 2, "q4_K", True, gb, ub, db)[0])
    return out


def test_golden_digests():
    """tests/golden/oracle_digests.json was written by tests/golden/make_golden.py on a
    machine where every digest's output had just been compared bit-for-bit with the
    reference library."""
    want = json.load(open(GOLDEN))
    got = _digest_cases()
    assert got["input_w"] == want["input_w"], "input generator drifted, not the oracle"
    assert got == want


def test_swiglu_oracle_is_silu_times_gate():
    """orc_swiglu against what the mathematics fixes: y * sigmoid(y) * z in float64, its values at
    0 and for large |y| (z y and 0), and its antisymmetry in z."""
    rng = np.random.default_rng(11)
    y = rng.normal(0, 3, 4096).astype(np.float32)
    z = rng.normal(0, 2, 4096).astype(np.float32)
    got = cr.swiglu(y, z)
    want = y.astype(np.float64) / (1.0 + np.exp(-y.astype(np.float64))) * z.astype(np.float64)
    assert np.abs(got - want).max() <= 4e-7 * np.abs(want).max()
    assert np.array_equal(cr.swiglu(np.zeros(4, np.float32), z[:4]), np.zeros(4, np.float32))
    big = np.array([40.0, -40.0, 100.0, -100.0], np.float32)
    assert np.allclose(cr.swiglu(big, np.full(4, 2.0, np.float32)), [80.0, 0.0, 200.0, 0.0], atol=1e-12)
    assert np.array_equal(cr.swiglu(y, -z), -got)
