"""GPU parity: mixture-of-experts block against the oracle (which restates
qwen_moe_layer.cpp:394-503 on top of the reference's M = 1 matmul arithmetic)."""
import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu


def _experts(cr, e, i, h, seed):
    gate, up, down = [], [], []
    for x in range(e):
        gate.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(seed + 3 * x, (i, h), 0.02)))
        up.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(seed + 3 * x + 1, (i, h), 0.02)))
        down.append(cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(seed + 3 * x + 2, (h, i), 0.02)))
    return gate, up, down


# the later shapes reach the kernels' other paths: 16- and 32-token work items with
# experts that hold more tokens than one item (48 tokens x 4 of 4 experts), long rows
# (hidden 3072 at 32 tokens), rows beyond what the matrix-core kernels stage in LDS
# (hidden 8192), and a block with enough work items for the plain (unpaired) gate/up
# form (64 tokens over 128 experts, 768 columns)
@pytest.mark.parametrize("t,h,i,e,k", [(8, 256, 256, 8, 2), (64, 512, 256, 16, 4), (5, 2048, 768, 8, 8),
                                       (40, 512, 256, 8, 2), (48, 256, 512, 4, 4), (72, 3072, 256, 4, 2),
                                       (3, 8192, 256, 4, 2), (64, 256, 768, 128, 8)])
def test_moe_matches_oracle(hipq, cr, t, h, i, e, k):
    import gpu_util as gu
    import torch
    gate, up, down = _experts(cr, e, i, h, seed=1000)
    x = synth.normal(2000, (t, h))
    logits = synth.normal(2001, (t, e))
    ref_y, ref_idx, ref_w = cr.moe_forward(x, logits, gate, up, down, k)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    dx, dl = gu.dev(x), gu.dev(logits)
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    wt = torch.zeros((t, k), device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, dx, y, router_logits=dl, topk_idx=idx, topk_w=wt,
                     stream=gu.stream())
    torch.cuda.synchronize()
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    assert np.abs(wt.cpu().numpy() - ref_w).max() <= 1e-6
    got = y.cpu().numpy()
    assert not np.isnan(got).any()
    # every single-row product carries the reference's bits; only the softmax
    # row sum (order unspecified in the reference, BLAS) may move the last bits
    assert gu.rel_err(got, ref_y) <= 2e-6, gu.rel_err(got, ref_y)
    # second call on the same handles (cached expert table) gives the same bits
    y2 = torch.empty_like(y)
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, dx, y2, router_logits=dl, stream=gu.stream())
    torch.cuda.synchronize()
    assert torch.equal(y, y2)
    for w in wg + wu + wd:
        w.destroy()


def test_moe_seeded_blocks(hipq, cr):
    """Twenty-four blocks drawn from a seeded generator: one to 130 tokens, 4 to 64 experts, top-1 to
    top-8, hidden sizes 256 to 2048, a third of them with one expert favoured by every token, every
    second one on a stream of its own. Expert choices identical, outputs within 2e-6."""
    import gpu_util as gu
    import torch
    rng = np.random.default_rng(5)
    cache = {}
    for it in range(24):
        h = int(rng.choice([256, 512, 1024, 2048]))
        i = int(rng.choice([256, 512, 768]))
        e = int(rng.choice([4, 8, 16, 32, 64]))
        k = min(int(rng.choice([1, 2, 4, 8])), e)
        t = int(rng.choice([1, 2, 3, 7, 8, 9, 16, 17, 31, 40, 64, 100, 130]))
        if (e, i, h) not in cache:
            if len(cache) > 4:
                cache.clear()
            cache[(e, i, h)] = _experts(cr, e, i, h, seed=100 + h)
        gate, up, down = cache[(e, i, h)]
        x = synth.normal(7000 + it, (t, h))
        logits = synth.normal(7100 + it, (t, e))
        if rng.random() < 0.3:
            logits[:, int(rng.integers(0, e))] += 6.0
        ref_y, ref_idx, _ = cr.moe_forward(x, logits, gate, up, down, k)
        wg = [capi.Weight("q4_K", i, h, b) for b in gate]
        wu = [capi.Weight("q4_K", i, h, b) for b in up]
        wd = [capi.Weight("q4_K", h, i, b) for b in down]
        dx, dl = gu.dev(x), gu.dev(logits)
        y = torch.full((t, h), float("nan"), device="cuda")
        idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
        st = torch.cuda.Stream() if it % 2 else torch.cuda.current_stream()
        torch.cuda.synchronize()
        capi.moe_forward(t, h, i, e, k, wg, wu, wd, dx, y, router_logits=dl, topk_idx=idx, stream=st.cuda_stream)
        torch.cuda.synchronize()
        case = (it, t, h, i, e, k)
        assert np.array_equal(idx.cpu().numpy(), ref_idx), case
        got = y.cpu().numpy()
        assert not np.isnan(got).any(), case
        assert gu.rel_err(got, ref_y) <= 2e-6, (case, gu.rel_err(got, ref_y))
        for w in wg + wu + wd:
            w.destroy()


@pytest.mark.parametrize("t,h,i,e,k", [(64, 512, 256, 32, 2), (64, 256, 256, 16, 2), (96, 256, 256, 8, 2)])
def test_moe_skewed_routing(hipq, cr, t, h, i, e, k):
    """Every token chooses expert 0: it holds far more slots than a work item (8, 16 or
    32 of them), so several workgroups serve it side by side."""
    import gpu_util as gu
    import torch
    gate, up, down = _experts(cr, e, i, h, seed=5000)
    x = synth.normal(5100, (t, h))
    logits = synth.normal(5101, (t, e))
    logits[:, 0] += 8.0
    ref_y, ref_idx, ref_w = cr.moe_forward(x, logits, gate, up, down, k)
    assert (ref_idx == 0).any(axis=1).all()
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, router_logits=gu.dev(logits), topk_idx=idx,
                     stream=gu.stream())
    torch.cuda.synchronize()
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    got = y.cpu().numpy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref_y) <= 2e-6, gu.rel_err(got, ref_y)
    for w in wg + wu + wd:
        w.destroy()


def test_moe_block_without_a_pair_sort_with_crowded_experts(hipq, cr):
    """40 tokens over 48 experts, 1024 intermediate columns: the regime in which the expert kernels
    find their pairs in the routing's output themselves. Expert 0 is chosen by every token (three
    chunks of 16, 16 and 8 pairs: the later rows of the grid), expert 1 by the first twelve (one
    chunk in the 16-row form), the others by a few (the 8-row form) or by none."""
    import gpu_util as gu
    import torch
    t, h, i, e, k = 40, 256, 1024, 48, 4
    gate, up, down = _experts(cr, e, i, h, seed=8000)
    x = synth.normal(8100, (t, h))
    logits = synth.normal(8101, (t, e))
    logits[:, 0] += 9.0
    logits[:12, 1] += 8.0
    logits[:, 40:] -= 20.0  # experts nobody chooses
    ref_y, ref_idx, ref_w = cr.moe_forward(x, logits, gate, up, down, k)
    counts = np.bincount(ref_idx.ravel(), minlength=e)
    assert counts[0] == 40 and 12 <= counts[1] <= 16 and (counts[40:] == 0).all() and (counts[2:40] <= 8).all()
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    for rep in range(2):  # the second call reuses the workspace the first one left
        y.fill_(float("nan"))
        capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, router_logits=gu.dev(logits), topk_idx=idx,
                         stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(idx.cpu().numpy(), ref_idx)
        got = y.cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, ref_y) <= 2e-6, gu.rel_err(got, ref_y)
    # the same block with every operand in host memory: the bits of the device-memory call
    yh = np.full((t, h), np.nan, np.float32)
    idxh = np.zeros((t, k), np.int32)
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, x, yh, router_logits=logits, topk_idx=idxh, mem=capi.MEM_HOST,
                     stream=gu.stream())
    assert np.array_equal(idxh, ref_idx)
    assert np.array_equal(yh.view(np.uint32), got.view(np.uint32))
    for w in wg + wu + wd:
        w.destroy()


def test_moe_long_chunk_uses_the_multi_kernel_sort(hipq, cr):
    """More than 16384 (token, expert) pairs: the pairs are counted, scanned and
    scattered by separate kernels, which also list the work items."""
    import gpu_util as gu
    import torch
    t, h, i, e, k = 2112, 256, 256, 8, 8
    gate, up, down = _experts(cr, e, i, h, seed=9000)
    x = synth.normal(9100, (t, h))
    logits = synth.normal(9101, (t, e))
    ref_y, ref_idx, _ = cr.moe_forward(x, logits, gate, up, down, k)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    y = torch.full((t, h), float("nan"), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, router_logits=gu.dev(logits), topk_idx=idx,
                     stream=gu.stream())
    torch.cuda.synchronize()
    assert np.array_equal(np.sort(idx.cpu().numpy(), axis=1), np.sort(ref_idx, axis=1))
    got = y.cpu().numpy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref_y) <= 2e-6, gu.rel_err(got, ref_y)
    for w in wg + wu + wd:
        w.destroy()


def test_expert_weights_serve_the_moe_block_only(hipq, cr):
    """Q4_K experts are re-stored for the expert kernels at the first block; a plain
    matmul on such a handle is refused, the block keeps giving the same bits."""
    import gpu_util as gu
    import torch
    t, h, i, e, k = 4, 256, 256, 4, 2
    gate, up, down = _experts(cr, e, i, h, seed=7000)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    x = gu.dev(synth.normal(7100, (t, h)))
    logits = gu.dev(synth.normal(7101, (t, e)))
    a = gu.dev(synth.normal(7102, (1, h)))
    c = torch.empty((1, i), device="cuda")
    capi.matmul(wg[0], a, 1, c, stream=gu.stream())  # fine before the first block
    y1, y2 = torch.empty((t, h), device="cuda"), torch.empty((t, h), device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, x, y1, router_logits=logits, stream=gu.stream())
    with pytest.raises(capi.HipqError):
        capi.matmul(wg[0], a, 1, c, stream=gu.stream())
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, x, y2, router_logits=logits, stream=gu.stream())
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)
    for w in wg + wu + wd:
        w.destroy()


@pytest.mark.parametrize("t", [1, 24])
def test_moe_block_replays_from_a_captured_graph(hipq, cr, t):
    """After a first call (which builds the expert table and the workspace) the block is
    kernel launches only: a caller can capture it. Every replay, with new inputs and
    other work in between, gives the bits of a direct call."""
    import gpu_util as gu
    import torch
    h, i, e, k = 512, 256, 16, 4
    gate, up, down = _experts(cr, e, i, h, seed=1500)
    ex = capi.Experts([capi.Weight("q4_K", i, h, b) for b in gate], [capi.Weight("q4_K", i, h, b) for b in up],
                      [capi.Weight("q4_K", h, i, b) for b in down])
    x = torch.zeros((t, h), device="cuda")
    logits = torch.zeros((t, e), device="cuda")
    y = torch.zeros((t, h), device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        capi.moe_forward(t, h, i, e, k, ex, None, None, x, y, router_logits=logits, stream=side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        capi.moe_forward(t, h, i, e, k, ex, None, None, x, y, router_logits=logits, stream=side.cuda_stream)
    for it in range(4):
        x.copy_(gu.dev(synth.normal(1510 + it, (t, h))))
        logits.copy_(gu.dev(synth.normal(1520 + it, (t, e))))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        other = torch.randn(1 << 20, device="cuda").sum()
        y.fill_(float("nan"))
        capi.moe_forward(t, h, i, e, k, ex, None, None, x, y, router_logits=logits, stream=gu.stream())
        torch.cuda.synchronize()
        assert torch.equal(got, y), "replay %d differs from the direct call" % it
        assert torch.isfinite(other)
    del graph
    for ws in ex.weights:
        for w in ws:
            w.destroy()


def test_moe_router_weight_path(hipq, cr):
    """Logits computed on the device from the fp32 router weight."""
    import gpu_util as gu
    import torch
    t, h, i, e, k = 6, 256, 256, 8, 2
    gate, up, down = _experts(cr, e, i, h, seed=3000)
    x = synth.normal(3100, (t, h))
    wr = synth.normal(3101, (h, e), 0.1)
    logits = cr.router_logits(x, wr, k)
    ref_y, ref_idx, _ = cr.moe_forward(x, logits, gate, up, down, k)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    y = torch.empty((t, h), device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), y, router_weight=gu.dev(wr), topk_idx=idx,
                     stream=gu.stream())
    torch.cuda.synchronize()
    assert np.array_equal(idx.cpu().numpy(), ref_idx)
    assert gu.rel_err(y.cpu().numpy(), ref_y) <= gu.TOL  # logits differ in the last bits only
    for w in wg + wu + wd:
        w.destroy()


@pytest.mark.parametrize("t,pinned", [(1, True), (5, True), (8, False), (9, False)])
def test_moe_decode_step_in_host_memory(hipq, cr, t, pinned):
    """A decode step's MoE block with x and y in host memory (page-locked: read and written where
    they lie; pageable: through the stream's staging buffer; nine tokens: through the copy engines):
    the bits of the device-memory call, with the router weight given in host memory."""
    import ctypes
    import gpu_util as gu
    import torch
    h, i, e, k = 512, 256, 8, 2
    gate, up, down = _experts(cr, e, i, h, seed=5200)
    wg = [capi.Weight("q4_K", i, h, b) for b in gate]
    wu = [capi.Weight("q4_K", i, h, b) for b in up]
    wd = [capi.Weight("q4_K", h, i, b) for b in down]
    x = synth.normal(5300 + t, (t, h))
    wr = synth.normal(5301, (h, e), 0.1)
    want = torch.full((t, h), float("nan"), device="cuda")
    capi.moe_forward(t, h, i, e, k, wg, wu, wd, gu.dev(x), want, router_weight=gu.dev(wr), stream=gu.stream())
    torch.cuda.synchronize()
    if pinned:
        px, py = capi.host_alloc(t * h * 4), capi.host_alloc(t * h * 4)
        xa = np.ctypeslib.as_array(ctypes.cast(px, ctypes.POINTER(ctypes.c_float)), (t, h))
        ya = np.ctypeslib.as_array(ctypes.cast(py, ctypes.POINTER(ctypes.c_float)), (t, h))
        xa[:] = x
        xin, yout = px, py
    else:
        ya = np.full((t, h), np.nan, np.float32)
        xin, yout = x, ya
    try:
        for _ in range(2):
            ya[:] = np.nan
            capi.moe_forward(t, h, i, e, k, wg, wu, wd, xin, yout, router_weight=wr, mem=capi.MEM_HOST)
            assert np.array_equal(ya.view(np.uint32), want.cpu().numpy().view(np.uint32))
    finally:
        if pinned:
            capi.host_free(px)
            capi.host_free(py)
        for w in wg + wu + wd:
            w.destroy()
