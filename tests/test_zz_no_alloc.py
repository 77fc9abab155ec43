"""hipq_matmul_noalloc (quantized activations in the library's fixed scratch array, no
device allocation inside the call) against hipq_matmul on the same inputs, through the
C ABI. Both enqueue the same kernels, so the outputs must be the same bits. Every case
makes two calls in a row, the second with a smaller input: the scratch keeps the first
call's contents and nothing of it may leak into the second result."""
import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu


def _pair(hipq, cr, kind, n, k, m_big, m_small):
    import torch
    import gpu_util as gu

    blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(900 + n, (n, k), 0.02))
    w = capi.Weight(kind, n, k, blocks)
    try:
        for call, m in enumerate((m_big, m_small)):
            a = synth.normal(910 + 7 * call + m, (m, k))
            da = gu.dev(a)
            want = torch.full((m, n), float("nan"), device="cuda", dtype=torch.float32)
            got = torch.full((m, n), float("nan"), device="cuda", dtype=torch.float32)
            capi.matmul(w, da, m, want, stream=gu.stream())
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            capi.matmul_noalloc(w, da, m, got, stream=gu.stream())
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
            g, r = got.cpu().numpy(), want.cpu().numpy()
            assert not np.isnan(g).any()
            assert np.array_equal(g.view(np.uint32), r.view(np.uint32)), (kind, m, gu.rel_err(g, r))
            if call == 1:
                ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
                assert gu.rel_err(g, ref) <= gu.TOL
    finally:
        w.destroy()


@pytest.mark.parametrize("kind", ["q4_0", "q4_K", "q6_K"])
@pytest.mark.parametrize("m_big,m_small", [(256, 37), (64, 5), (6, 1)])
def test_noalloc_matches_matmul_twice(hipq, cr, kind, m_big, m_small):
    _pair(hipq, cr, kind, 640, 1024, m_big, m_small)


def test_noalloc_large_row_count_then_one_row(hipq, cr):
    """A vocabulary-sized matrix (two launches even for one row: the row's blocks pass
    through the scratch) after a prefill-sized call."""
    _pair(hipq, cr, "q4_K", 40000, 512, 512, 1)


def test_noalloc_rejects_what_does_not_fit(hipq, cr):
    import torch
    n, k = 256, 4096
    blocks = cr.quantize_weights(cr.oracle(), "q6_K", synth.normal(5, (n, k), 0.02))
    w = capi.Weight("q6_K", n, k, blocks)
    m = 4096  # 16.8 million values: beyond the scratch
    a = torch.zeros((m, k), device="cuda")
    c = torch.zeros((m, n), device="cuda")
    with pytest.raises(capi.HipqError) as e:
        capi.matmul_noalloc(w, a, m, c)
    assert e.value.code == -4 and "scratch" in str(e.value)
    w.destroy()


def test_noalloc_q6_K_prefill_before_the_tile_copy_exists(hipq, cr):
    """The Q6_K matrix-core product needs the weight's tile copy, which only an allocating call can
    build: on a fresh weight the allocation-free call walks the rows through the GEMV engine
    (the reference's bits); once hipq_matmul has built the copy both calls run the same kernel."""
    import torch
    import gpu_util as gu
    n, k, m = 320, 512, 40
    blocks = cr.quantize_weights(cr.oracle(), "q6_K", synth.normal(77, (n, k), 0.02))
    w = capi.Weight("q6_K", n, k, blocks)
    try:
        a = synth.normal(78, (m, k))
        da = gu.dev(a)
        ref = cr.gemm(cr.oracle(), "q6_K", a, blocks, n)
        first = torch.full((m, n), float("nan"), device="cuda")
        free_before = torch.cuda.mem_get_info()[0]
        capi.matmul_noalloc(w, da, m, first, stream=gu.stream())
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert np.array_equal(first.cpu().numpy().view(np.uint32), ref.view(np.uint32))
        full = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul(w, da, m, full, stream=gu.stream())
        again = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul_noalloc(w, da, m, again, stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(again.cpu().numpy(), full.cpu().numpy())
        assert gu.rel_err(full.cpu().numpy(), ref) <= gu.TOL
    finally:
        w.destroy()


def test_noalloc_q4_K_few_rows_before_and_after_the_tile_copy(hipq, cr):
    """Five to eight rows of a Q4_K matrix run on the matrix cores off the weight's tile copy, which
    only an allocating call can build: on a fresh weight the allocation-free call takes the GEMV
    engine, afterwards the matrix-core kernel. Both carry the reference's bits."""
    import torch
    import gpu_util as gu
    n, k, m = 1056, 1024, 6
    blocks = cr.quantize_weights(cr.oracle(), "q4_K", synth.normal(87, (n, k), 0.02))
    w = capi.Weight("q4_K", n, k, blocks)
    try:
        a = synth.normal(88, (m, k))
        da = gu.dev(a)
        ref = cr.gemm(cr.oracle(), "q4_K", a, blocks, n)
        first = torch.full((m, n), float("nan"), device="cuda")
        free_before = torch.cuda.mem_get_info()[0]
        capi.matmul_noalloc(w, da, m, first, stream=gu.stream())
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert np.array_equal(first.cpu().numpy().view(np.uint32), ref.view(np.uint32))
        full = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul(w, da, m, full, stream=gu.stream())
        again = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul_noalloc(w, da, m, again, stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(full.cpu().numpy().view(np.uint32), ref.view(np.uint32))
        assert np.array_equal(again.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    finally:
        w.destroy()



def test_noalloc_in_parts_of_k_matches_matmul(hipq, cr):
    """Few tiles and K >= 2048: hipq_matmul forms such a Q4_K / Q6_K product in parts of K once the
    weight has its tile copy. The allocation-free call does the same when the parts' partial sums fit
    its slot beside the activations (same kernels, same bits); with C at an address or pitch that
    rules the parts out, both entry points take whole rows and agree with the parts to 1e-4."""
    import torch
    import gpu_util as gu
    for kind in ("q4_K", "q6_K"):
        n, k, m = 1024, 2048, 64
        blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(97, (n, k), 0.02))
        w = capi.Weight(kind, n, k, blocks)
        try:
            a = synth.normal(98, (m, k))
            da = gu.dev(a)
            ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
            full = torch.full((m, n), float("nan"), device="cuda")
            capi.matmul(w, da, m, full, stream=gu.stream())      # builds the tile copy, then parts of K
            again = torch.full((m, n), float("nan"), device="cuda")
            capi.matmul(w, da, m, again, stream=gu.stream())
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            got = torch.full((m, n), float("nan"), device="cuda")
            capi.matmul_noalloc(w, da, m, got, stream=gu.stream())
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before
            assert np.array_equal(full.cpu().numpy(), again.cpu().numpy())
            assert np.array_equal(got.cpu().numpy().view(np.uint32), full.cpu().numpy().view(np.uint32)), kind
            assert gu.rel_err(got.cpu().numpy(), ref) <= gu.TOL
            # a pitch that is no multiple of four: whole rows for both entry points
            wide_a = torch.full((m, n + 1), float("nan"), device="cuda")
            wide_b = torch.full((m, n + 1), float("nan"), device="cuda")
            capi.matmul(w, da, m, wide_a, ldc=n + 1, stream=gu.stream())
            capi.matmul_noalloc(w, da, m, wide_b, ldc=n + 1, stream=gu.stream())
            torch.cuda.synchronize()
            ga, gb = wide_a.cpu().numpy()[:, :n], wide_b.cpu().numpy()[:, :n]
            assert np.array_equal(ga.view(np.uint32), gb.view(np.uint32))
            assert gu.rel_err(ga, ref) <= gu.TOL and gu.rel_err(ga, full.cpu().numpy()) <= gu.TOL
        finally:
            w.destroy()


def test_noalloc_streams_have_their_own_slots(hipq, cr):
    """Every stream that uses the entry point gets a slot of the fixed array of its own: calls queued
    on two streams at once (different weights and row counts, so different scratch contents) give
    what each gives alone; a fifth stream is refused until a slot has been released."""
    import torch
    import gpu_util as gu
    n, k = 768, 1024
    ws, acts, wants = [], [], []
    for j, (kind, m) in enumerate((("q4_K", 96), ("q6_K", 40), ("q4_0", 128))):
        blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(120 + j, (n, k), 0.02))
        ws.append(capi.Weight(kind, n, k, blocks))
        a = synth.normal(130 + j, (m, k))
        acts.append((gu.dev(a), m))
        want = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul(ws[-1], acts[-1][0], m, want, stream=gu.stream())
        wants.append(want)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(3)]
    try:
        gots = [torch.full_like(x, float("nan")) for x in wants]
        for rounds in range(3):  # several calls in flight on every stream
            for j, st in enumerate(streams):
                capi.matmul_noalloc(ws[j], acts[j][0], acts[j][1], gots[j], stream=st.cuda_stream)
        torch.cuda.synchronize()
        for j in range(3):
            assert np.array_equal(gots[j].cpu().numpy().view(np.uint32), wants[j].cpu().numpy().view(np.uint32)), j
        # the test stream may hold the fourth slot already; two more streams exhaust the array
        extra = [torch.cuda.Stream() for _ in range(2)]
        codes = []
        for st in extra:
            try:
                capi.matmul_noalloc(ws[0], acts[0][0], acts[0][1], gots[0], stream=st.cuda_stream)
                codes.append(0)
            except capi.HipqError as e:
                codes.append(e.code)
                assert "slot" in str(e)
        torch.cuda.synchronize()
        assert codes[-1] == -4, codes
        capi.stream_release(streams[2].cuda_stream)     # gives a slot back
        capi.matmul_noalloc(ws[0], acts[0][0], acts[0][1], gots[0], stream=extra[-1].cuda_stream)
        torch.cuda.synchronize()
        assert np.array_equal(gots[0].cpu().numpy().view(np.uint32), wants[0].cpu().numpy().view(np.uint32))
        for st in extra:
            capi.stream_release(st.cuda_stream)
    finally:
        for st in streams:
            capi.stream_release(st.cuda_stream)
        for w in ws:
            w.destroy()
