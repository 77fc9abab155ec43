"""GPU parity of product branches the other files do not reach: the MoE block with the
softmax values used as they are (renormalize = 0, the reference's forwarding path,
qwen_moe_layer.cpp:161-259), MoE blocks whose experts are Q4_0 or Q6_K (MoELayer accepts
any weight dtype of the model, qwen_moe_layer.cpp:50-159), and Q4_0 matmuls whose K is a
multiple of 32 but not of 256 (legal per q4_0_tensor.cpp:25-28). All against the oracle,
through the C ABI."""
import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu


def _experts(cr, kind, e, i, h, seed):
    q = lambda s, shape: cr.quantize_weights(cr.oracle(), kind, synth.normal(s, shape, 0.02))
    return ([q(seed + 3 * x, (i, h)) for x in range(e)], [q(seed + 3 * x + 1, (i, h)) for x in range(e)],
            [q(seed + 3 * x + 2, (h, i)) for x in range(e)])


def _run_moe(cr, kind, t, h, i, e, k, renormalize, seed):
    import gpu_util as gu
    import torch
    gate, up, down = _experts(cr, kind, e, i, h, seed)
    x = synth.normal(seed + 500, (t, h))
    logits = synth.normal(seed + 501, (t, e))
    ref_y, ref_idx, ref_w = cr.moe_forward(x, logits, gate, up, down, k, kind=kind, renormalize=renormalize)
    wg = [capi.Weight(kind, i, h, b) for b in gate]
    wu = [capi.Weight(kind, i, h, b) for b in up]
    wd = [capi.Weight(kind, h, i, b) for b in down]
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    wt = torch.zeros((t, k), device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, router_logits=gu.dev(logits), topk_idx=idx,
                     topk_w=wt, renormalize=renormalize, stream=gu.stream())
    torch.cuda.synchronize()
    for w in wg + wu + wd:
        w.destroy()
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    assert np.abs(wt.cpu().numpy() - ref_w).max() <= 1e-6
    if not renormalize:
        assert (ref_w.sum(1) < 0.999).all(), "the case must tell the two weightings apart"
    got = y.cpu().numpy()
    assert not np.isnan(got).any()
    # every single-row product carries the reference's bits; only the softmax row sum
    # (order unspecified in the reference) may move the last bits of the routing weights
    assert gu.rel_err(got, ref_y) <= 2e-6, gu.rel_err(got, ref_y)


@pytest.mark.parametrize("t,h,i,e,k", [(8, 256, 256, 8, 2), (64, 512, 256, 16, 4), (1, 2048, 768, 16, 8)])
def test_moe_without_renormalization(hipq, cr, t, h, i, e, k):
    _run_moe(cr, "q4_K", t, h, i, e, k, False, seed=7000)


@pytest.mark.parametrize("kind", ["q4_0", "q6_K"])
@pytest.mark.parametrize("t,h,i,e,k,renorm", [(6, 256, 256, 8, 2, True), (33, 512, 256, 8, 4, True),
                                              (1, 1024, 512, 4, 2, True), (12, 256, 512, 8, 3, False)])
def test_moe_with_q4_0_and_q6_K_experts(hipq, cr, kind, t, h, i, e, k, renorm):
    _run_moe(cr, kind, t, h, i, e, k, renorm, seed=7100)


@pytest.mark.parametrize("k", [32, 96, 1056])
@pytest.mark.parametrize("m", [1, 5, 64])
def test_q4_0_with_k_not_a_multiple_of_256(hipq, cr, k, m):
    import gpu_util as gu
    n = 320
    blocks = cr.quantize_weights(cr.oracle(), "q4_0", synth.normal(7200 + k, (n, k), 0.02))
    a = synth.normal(7300 + m, (m, k))
    ref = cr.gemm(cr.oracle(), "q4_0", a, blocks, n)
    w = capi.Weight("q4_0", n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_router_with_nan_logits_stays_in_range(hipq, cr):
    """A NaN among the router logits must still give expert indices below E (the reference's
    partial_sort always does): the expert kernels index tables with them."""
    import gpu_util as gu
    import torch
    t, h, i, e, k = 4, 256, 256, 8, 2
    gate, up, down = _experts(cr, "q4_K", e, i, h, 7400)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    logits = synth.normal(7401, (t, e))
    logits[1, :] = np.nan
    logits[2, 3] = np.nan
    y = torch.zeros((t, h), device="cuda")
    idx = torch.full((t, k), -1, dtype=torch.int32, device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(synth.normal(7402, (t, h))), y, router_logits=gu.dev(logits),
                     topk_idx=idx, stream=gu.stream())
    torch.cuda.synchronize()
    got = idx.cpu().numpy()
    for w in wg + wu + wd:
        w.destroy()
    assert ((got >= 0) & (got < e)).all(), got
    assert all(len(set(r)) == k for r in got.tolist())


def _gpt_oss_case(cr, kind, t, h, i, e, k, seed):
    gate, up, down = _experts(cr, kind, e, i, h, seed)
    x = synth.normal(seed + 500, (t, h))
    gb = synth.normal(seed + 502, (e, i), 0.3)
    ub = synth.normal(seed + 503, (e, i), 0.3)
    db = synth.normal(seed + 504, (e, h), 0.3)
    return gate, up, down, x, gb, ub, db


@pytest.mark.parametrize("kind,t,h,i,e,k", [("q4_K", 8, 256, 256, 8, 2), ("q4_K", 64, 512, 256, 16, 4),
                                            ("q4_K", 1, 2048, 768, 16, 4), ("q4_0", 9, 256, 512, 8, 4),
                                            ("q6_K", 5, 512, 256, 4, 2),
                                            # 40 tokens over 48 experts and 1024 columns: the block without a pair sort
                                            ("q4_K", 40, 256, 1024, 48, 4)])
def test_gpt_oss_moe_matches_oracle(hipq, cr, kind, t, h, i, e, k):
    """hipq_moe_forward_ext, GPT-OSS variant (gpt_oss_moe_layer.cpp:372-449, 452-568): biased
    projections, swiglu with alpha on (gate, up + 1), biased down projection. The integer and
    fp32 chains of the three products carry the reference's bits; the exponential is the device's
    expf against the host's, so the bar is the fp32 tolerance, not bit identity."""
    import gpu_util as gu
    import torch
    gate, up, down, x, gb, ub, db = _gpt_oss_case(cr, kind, t, h, i, e, k, 7600)
    logits = synth.normal(7601, (t, e))
    ref_y, ref_idx, ref_w = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k, kind=kind)
    wg = [capi.Weight(kind, i, h, b) for b in gate]
    wu = [capi.Weight(kind, i, h, b) for b in up]
    wd = [capi.Weight(kind, h, i, b) for b in down]
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    capi.moe_forward_gpt_oss(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, gu.dev(gb), gu.dev(ub), gu.dev(db),
                             router_logits=gu.dev(logits), topk_idx=idx, stream=gu.stream())
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref_y) <= gu.TOL, gu.rel_err(got, ref_y)
    # the biases and the + 1 matter at this size: without them the result is far off
    plain, _, _ = cr.moe_forward(x, logits, gate, up, down, k, kind=kind)
    assert gu.rel_err(plain, ref_y) > 0.05
    for w in wg + wu + wd:
        w.destroy()


def test_gpt_oss_moe_router_bias_and_host_memory(hipq, cr):
    """Router logits formed on the device from the fp32 router weight plus its bias
    (gpt_oss_moe_layer.cpp:500-503), all operands in host memory."""
    import gpu_util as gu
    kind, t, h, i, e, k = "q4_K", 6, 256, 256, 8, 2
    gate, up, down, x, gb, ub, db = _gpt_oss_case(cr, kind, t, h, i, e, k, 7700)
    wr = synth.normal(7701, (h, e), 0.1)
    rb = synth.normal(7702, (e,), 2.0)  # large enough to change the routing
    logits = cr.router_logits(x, wr, k, rb)
    ref_y, ref_idx, _ = cr.moe_forward_gpt_oss(x, logits, gate, up, down, gb, ub, db, k, kind=kind)
    _, idx_without, _ = cr.moe_forward_gpt_oss(x, logits - rb, gate, up, down, gb, ub, db, k, kind=kind)
    assert not np.array_equal(ref_idx, idx_without), "the bias must change the routing of the case"
    wg = [capi.Weight(kind, i, h, b) for b in gate]
    wu = [capi.Weight(kind, i, h, b) for b in up]
    wd = [capi.Weight(kind, h, i, b) for b in down]
    y = np.full((t, h), np.nan, np.float32)
    idx = np.zeros((t, k), np.int32)
    capi.moe_forward_gpt_oss(t, h, i, e, k, wg, wu, wd, x, y, gb, ub, db, router_weight=wr, router_bias=rb,
                             topk_idx=idx, mem=capi.MEM_HOST)
    assert np.array_equal(idx, ref_idx)
    assert gu.rel_err(y, ref_y) <= gu.TOL  # logits differ in the last bits only
    with pytest.raises(capi.HipqError):  # a bias for logits the caller computed is refused
        capi.moe_forward_gpt_oss(t, h, i, e, k, wg, wu, wd, x, y, gb, ub, db, router_logits=logits, router_bias=rb,
                                 mem=capi.MEM_HOST)
    for w in wg + wu + wd:
        w.destroy()


@pytest.mark.parametrize("kind,m,k,n,nd", [("q4_0", 1, 1024, 3072, 1024), ("q4_K", 1, 2048, 768, 2048),
                                           ("q6_K", 3, 512, 256, 512), ("q4_0", 24, 1024, 3072, 1024),
                                           ("q4_K", 5, 1024, 512, 768), ("q4_K", 80, 1024, 1024, 512),
                                           ("q4_0", 1, 96, 320, 64)])
@pytest.mark.parametrize("mem", ["device", "host"])
def test_mlp_swiglu_down_is_the_two_calls_and_matches_the_oracle(hipq, cr, kind, m, k, n, nd, mem):
    """hipq_mlp_swiglu_down: out = swiglu(a . Wup^T, a . Wgate^T) . Wdown^T, the four layers of
    CausalLM::createMlp (causal_lm.cpp:671-705) as one call. Bit for bit what hipq_mlp_swiglu followed by
    hipq_matmul give, and within the fp32 tolerance of the oracle's products, its swiglu and its down
    product on the oracle's own hidden rows."""
    import gpu_util as gu
    import torch
    wa = cr.quantize_weights(cr.oracle(), kind, synth.normal(8800 + n, (n, k), 0.05))
    wm = cr.quantize_weights(cr.oracle(), kind, synth.normal(8801 + n, (n, k), 0.05))
    wd = cr.quantize_weights(cr.oracle(), kind, synth.normal(8802 + n, (nd, n), 0.05))
    a = synth.normal(8803 + m, (m, k))
    hidden = cr.swiglu(cr.gemm(cr.oracle(), kind, a, wa, n), cr.gemm(cr.oracle(), kind, a, wm, n))
    ref = cr.gemm(cr.oracle(), kind, hidden, wd, nd)
    ha, hm, hd = capi.Weight(kind, n, k, wa), capi.Weight(kind, n, k, wm), capi.Weight(kind, nd, n, wd)
    try:
        two = torch.full((m, nd), float("nan"), device="cuda")
        h = torch.full((m, n), float("nan"), device="cuda")
        capi.mlp_swiglu(ha, hm, gu.dev(a), m, h, stream=gu.stream())
        capi.matmul(hd, h, m, two, stream=gu.stream())
        torch.cuda.synchronize()
        if mem == "device":
            ldo = nd + 4
            out = torch.full((m, ldo), float("nan"), device="cuda")
            capi.mlp_swiglu_down(ha, hm, hd, gu.dev(a), m, out, ldo=ldo, stream=gu.stream())
            torch.cuda.synchronize()
            assert torch.isnan(out[:, nd:]).all(), "the call wrote between the rows of the output"
            got = out[:, :nd].cpu().numpy()
        else:
            got = np.full((m, nd), np.nan, np.float32)
            capi.mlp_swiglu_down(ha, hm, hd, a, m, got, mem=capi.MEM_HOST)
        assert not np.isnan(got).any()
        assert np.array_equal(got.view(np.uint32), two.cpu().numpy().view(np.uint32))
        assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
        if k != n:
            with pytest.raises(capi.HipqError):   # a down projection that does not fit the hidden rows
                capi.mlp_swiglu_down(ha, hm, ha, gu.dev(a), m, two, stream=gu.stream())
    finally:
        for w in (ha, hm, hd):
            w.destroy()


@pytest.mark.parametrize("kind,m,k,n", [("q4_0", 1, 1024, 3072), ("q4_K", 1, 2048, 768), ("q6_K", 1, 1024, 512),
                                        ("q4_0", 1, 96, 320),      # K below one chunk unit: not fused
                                        ("q4_0", 24, 1024, 3072), ("q4_K", 5, 1024, 512),
                                        # one row, the row length a constant of the launch (4096, 3072) or not (2304),
                                        # the weights asked for in front of, behind and around the row's quantization
                                        ("q4_K", 1, 4096, 2200), ("q4_K", 1, 3072, 3000), ("q6_K", 1, 4096, 1100),
                                        ("q4_0", 1, 4096, 2100), ("q4_K", 1, 2304, 1000), ("q4_K", 1, 2048, 4100)])
@pytest.mark.parametrize("mem", ["device", "host"])
def test_mlp_swiglu_matches_oracle(hipq, cr, kind, m, k, n, mem):
    """hipq_mlp_swiglu: out = swiglu(a . Wact^T, a . Wmul^T) (swiglu.cpp:40-62 on the outputs of
    ffn_up and ffn_gate, causal_lm.cpp:672-695). The products carry the bits of hipq_matmul; the
    exponential is the device's, so the result is held to the fp32 tolerance."""
    import gpu_util as gu
    import torch
    wa = cr.quantize_weights(cr.oracle(), kind, synth.normal(7800 + n, (n, k), 0.05))
    wm = cr.quantize_weights(cr.oracle(), kind, synth.normal(7801 + n, (n, k), 0.05))
    a = synth.normal(7802 + m, (m, k))
    y = cr.gemm(cr.oracle(), kind, a, wa, n)
    z = cr.gemm(cr.oracle(), kind, a, wm, n)
    ref = cr.swiglu(y, z)
    assert np.abs(ref - y * z).max() > 0.05 * np.abs(ref).max(), "the activation must matter in this case"
    ha, hm = capi.Weight(kind, n, k, wa), capi.Weight(kind, n, k, wm)
    if mem == "device":
        out = torch.full((m, n), float("nan"), device="cuda")
        capi.mlp_swiglu(ha, hm, gu.dev(a), m, out, stream=gu.stream())
        torch.cuda.synchronize()
        got = out.cpu().numpy()
    else:
        got = np.full((m, n), np.nan, np.float32)
        capi.mlp_swiglu(ha, hm, a, m, got, mem=capi.MEM_HOST)
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
    # and it is the activation of the library's own products, element by element
    yg, zg = gu.gpu_matmul(ha, a), gu.gpu_matmul(hm, a)
    assert np.abs(got - cr.swiglu(yg, zg)).max() <= 1e-6 * np.abs(ref).max()
    ha.destroy()
    hm.destroy()
