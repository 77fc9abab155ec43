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

