"""Host-memory operands of the C ABI (HIPQ_MEM_HOST): pageable memory goes through the library's
pinned staging ring, page-locked memory (hipq_host_alloc, what the context's MemAllocator hands
the framework, cl_context.cpp:83) by DMA as it is. Both must give the bits of the device-memory
call. Also: the multi-weight call on host memory, and releasing a stream's scratch."""
import ctypes

import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu


def _device_result(w, a):
    import gpu_util as gu
    return gu.gpu_matmul(w, a)


@pytest.mark.parametrize("kind,m,k,n,lda_pad,ldc_pad", [
    ("q4_0", 700, 1024, 3000, 0, 0),     # A 2.8 MB, C 8.4 MB: several slices of the ring each way
    ("q4_0", 700, 1024, 3000, 32, 8),    # strided rows on both sides
    ("q4_K", 37, 2048, 1024, 0, 0),
    ("q6_K", 1, 1024, 5000, 0, 0),       # decode row
    ("q4_0", 1, 32, 600000, 0, 0),       # one output row longer than a ring slot (2.4 MB)
])
def test_pageable_operands_give_the_device_bits(hipq, cr, kind, m, k, n, lda_pad, ldc_pad):
    blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(9000 + n % 97, (n, k), 0.02))
    w = capi.Weight(kind, n, k, blocks)
    a = synth.normal(9001 + m, (m, k))
    want = _device_result(w, a)
    lda, ldc = k + lda_pad, n + ldc_pad
    a_host = np.full((m, lda), np.float32(7e9))
    a_host[:, :k] = a
    c_host = np.full((m, ldc), np.float32(-3.5))
    for _ in range(2):  # the second call finds ring slots and operand buffers in use before
        c_host[:, :n] = np.nan
        capi.matmul(w, a_host, m, c_host, lda=lda, ldc=ldc, mem=capi.MEM_HOST)
        assert np.array_equal(c_host[:, :n].view(np.uint32), want.view(np.uint32))
        assert np.all(c_host[:, n:] == np.float32(-3.5)), "the padding of the output rows was written"
    w.destroy()


def test_page_locked_operands(hipq, cr):
    kind, m, k, n = "q4_K", 64, 1024, 768
    blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(9100, (n, k), 0.02))
    w = capi.Weight(kind, n, k, blocks)
    a = synth.normal(9101, (m, k))
    want = _device_result(w, a)
    pa, pc = capi.host_alloc(m * k * 4), capi.host_alloc(m * n * 4)
    try:
        a_pin = np.ctypeslib.as_array(ctypes.cast(pa, ctypes.POINTER(ctypes.c_float)), (m, k))
        c_pin = np.ctypeslib.as_array(ctypes.cast(pc, ctypes.POINTER(ctypes.c_float)), (m, n))
        assert not a_pin.any() and not c_pin.any(), "the allocator hands out zero-filled memory"
        a_pin[:] = a
        capi.matmul(w, pa, m, pc, mem=capi.MEM_HOST)
        assert np.array_equal(c_pin.view(np.uint32), want.view(np.uint32))
    finally:
        capi.host_free(pa)
        capi.host_free(pc)
        capi.host_free(None)
    w.destroy()


@pytest.mark.parametrize("kind,m", [("q4_0", 1), ("q4_0", 19), ("q4_K", 1), ("q6_K", 3)])
def test_multi_weight_call_on_host_memory(hipq, cr, kind, m):
    """hipq_matmul_multi with host operands: the activation crosses once and the products run as
    for device memory; same bits as one hipq_matmul per weight."""
    k, ns = 1024, (512, 256, 384)
    ws = [capi.Weight(kind, n, k, cr.quantize_weights(cr.oracle(), kind, synth.normal(9200 + n, (n, k), 0.02)))
          for n in ns]
    a = synth.normal(9201 + m, (m, k))
    cs = [np.full((m, n), np.nan, np.float32) for n in ns]
    capi.matmul_multi(ws, a, m, cs, mem=capi.MEM_HOST)
    for w, c in zip(ws, cs):
        assert np.array_equal(c.view(np.uint32), _device_result(w, a).view(np.uint32))
        w.destroy()


def test_stream_release(hipq, cr):
    """A stream's scratch can be given back and comes again with the next call."""
    import gpu_util as gu
    import torch
    kind, m, k, n = "q4_K", 16, 1024, 512
    w = capi.Weight(kind, n, k, cr.quantize_weights(cr.oracle(), kind, synth.normal(9300, (n, k), 0.02)))
    a = synth.normal(9301, (m, k))
    want = _device_result(w, a)
    st = torch.cuda.Stream()
    da = gu.dev(a)
    torch.cuda.synchronize()
    for _ in range(2):
        dc = torch.full((m, n), float("nan"), device="cuda")
        torch.cuda.synchronize()
        capi.matmul(w, da, m, dc, stream=st.cuda_stream)
        st.synchronize()
        assert np.array_equal(dc.cpu().numpy().view(np.uint32), want.view(np.uint32))
        capi.stream_release(st.cuda_stream)
    capi.stream_release(st.cuda_stream)  # nothing kept: a no-op
    w.destroy()


class _Pinned:
    """A float32 array in page-locked memory of the context's allocator."""

    def __init__(self, shape, fill=None):
        self.n = int(np.prod(shape))
        self.addr = capi.host_alloc(self.n * 4)
        self.arr = np.ctypeslib.as_array(ctypes.cast(self.addr, ctypes.POINTER(ctypes.c_float)), tuple(shape))
        if fill is not None:
            self.arr[...] = fill

    def free(self):
        capi.host_free(self.addr)


@pytest.mark.parametrize("kind,m,k,n,lda_pad,ldc_pad", [
    ("q4_0", 1, 1024, 3072, 0, 0),      # one launch that quantizes the row itself
    ("q4_K", 1, 4096, 4096, 0, 0),
    ("q6_K", 1, 1024, 40000, 0, 0),     # two launches (vocabulary-sized)
    ("q4_K", 3, 2048, 1024, 8, 4),      # strided rows on both sides
    ("q4_0", 8, 1024, 3072, 0, 12),
    ("q4_K", 8, 4096, 12288, 0, 0),     # the few-rows matrix-core kernel
    ("q4_0", 9, 1024, 3072, 0, 0),
    ("q4_K", 64, 4096, 4096, 0, 8),     # a short prefill chunk: 1 MiB each way
    ("q6_K", 100, 1024, 2048, 4, 0),
    ("q4_0", 128, 1024, 3072, 0, 0),    # the most rows this path takes
    ("q4_0", 129, 1024, 3072, 0, 0),    # one row more: through the copy engines
    ("q4_0", 100, 1024, 8192, 0, 0),    # outputs beyond 2 MiB: through the copy engines
])
def test_a_few_page_locked_rows_take_no_copy(hipq, cr, kind, m, k, n, lda_pad, ldc_pad):
    """Up to 128 rows and 2 MiB a side in page-locked memory (a decode step or a short chunk through the
    Layer API): the rows are
    fetched by a kernel and the product kernels write the host tensor directly. Same bits as the
    device-memory call; the padding of strided rows stays untouched; two calls in a row."""
    blocks = cr.quantize_weights(cr.oracle(), kind, synth.normal(9400 + n % 89, (n, k), 0.02))
    w = capi.Weight(kind, n, k, blocks)
    a = synth.normal(9401 + m, (m, k))
    want = _device_result(w, a)
    lda, ldc = k + lda_pad, n + ldc_pad
    pa, pc = _Pinned((m, lda), 7e9), _Pinned((m, ldc), -3.5)
    try:
        pa.arr[:, :k] = a
        for _ in range(2):
            pc.arr[:, :n] = np.nan
            capi.matmul(w, pa.addr, m, pc.addr, lda=lda, ldc=ldc, mem=capi.MEM_HOST)
            assert np.array_equal(pc.arr[:, :n].view(np.uint32), want.view(np.uint32))
            assert np.all(pc.arr[:, n:] == np.float32(-3.5))
        # the rows of a decode step of a batch: each with the bits of its own one-row product
        pc.arr[:, :n] = np.nan
        capi.matmul_each_row(w, pa.addr, m, pc.addr, lda=lda, ldc=ldc, mem=capi.MEM_HOST)
        for r in range(m):
            assert np.array_equal(pc.arr[r, :n].view(np.uint32), _device_result(w, a[r:r + 1])[0].view(np.uint32)), r
    finally:
        pa.free()
        pc.free()
        w.destroy()


@pytest.mark.parametrize("kind,m", [("q4_0", 1), ("q4_K", 1), ("q4_0", 4), ("q4_K", 8), ("q6_K", 2)])
def test_grouped_calls_on_a_few_page_locked_rows(hipq, cr, kind, m):
    """hipq_matmul_multi (Q, K, V) and hipq_mlp_swiglu (up, gate and the activation) with a decode
    step's page-locked operands: outputs written by the kernels, the bits of the device calls."""
    import gpu_util as gu
    import torch
    k, ns = 1024, (2048, 1024, 1024)
    ws = [capi.Weight(kind, n, k, cr.quantize_weights(cr.oracle(), kind, synth.normal(9500 + j, (n, k), 0.05)))
          for j, n in enumerate(ns)]
    a = synth.normal(9510 + m, (m, k))
    pa = _Pinned((m, k), a)
    pcs = [_Pinned((m, n), np.nan) for n in ns]
    po = _Pinned((m, ns[1]), np.nan)
    try:
        capi.matmul_multi(ws, pa.addr, m, [p.addr for p in pcs], mem=capi.MEM_HOST)
        dev = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
        capi.matmul_multi(ws, gu.dev(a), m, dev, stream=gu.stream())
        torch.cuda.synchronize()
        for p, d in zip(pcs, dev):
            assert np.array_equal(p.arr.view(np.uint32), d.cpu().numpy().view(np.uint32))
        capi.mlp_swiglu(ws[1], ws[2], pa.addr, m, po.addr, mem=capi.MEM_HOST)
        want = torch.full((m, ns[1]), float("nan"), device="cuda")
        capi.mlp_swiglu(ws[1], ws[2], gu.dev(a), m, want, stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(po.arr.view(np.uint32), want.cpu().numpy().view(np.uint32))
        # the whole MLP in one call: the hidden rows stay on the device, the output is written in place
        capi.mlp_swiglu_down(ws[1], ws[2], ws[0], pa.addr, m, pcs[0].addr, mem=capi.MEM_HOST)
        whole = torch.full((m, ns[0]), float("nan"), device="cuda")
        capi.matmul(ws[0], want, m, whole, stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(pcs[0].arr.view(np.uint32), whole.cpu().numpy().view(np.uint32))
    finally:
        for p in [pa, po] + pcs:
            p.free()
        for w in ws:
            w.destroy()


@pytest.mark.parametrize("kind,m,k,n,pad", [
    ("q4_0", 1400, 1024, 3072, 0),      # five steps of 256 rows, the last of 376
    ("q4_0", 2100, 1024, 2048, 8),      # eight steps; strided rows on both sides
    ("q4_K", 700, 2048, 12288, 0),      # every step takes the prefill GEMM on whole K: two steps
    ("q4_K", 1100, 2048, 4096, 0),      # a step would run in parts of K (other bits): one piece
    ("q6_K", 1100, 1024, 4096, 4),
    ("q4_0", 512, 1024, 3072, 0),       # outputs of 6 MB: one piece
])
def test_prefill_rows_in_steps_give_the_device_bits(hipq, cr, kind, m, k, n, pad):
    """512 rows and more in page-locked memory with outputs of 16 MiB and at least twice the input cross in
    steps of 256: a step's rows come in and the step before goes out while the kernels work. Every entry point that takes host rows gives the bits of its
    device-memory call on the whole matrix, twice in a row."""
    import gpu_util as gu
    import torch
    nd = 1024
    mk = lambda j, rows, cols: capi.Weight(kind, rows, cols, cr.quantize_weights(
        cr.oracle(), kind, synth.normal(9700 + j, (rows, cols), 0.05)))
    w, w2, wd = mk(0, n, k), mk(1, n, k), mk(2, nd, n)
    a = synth.normal(9710 + m, (m, k))
    lda, ldc = k + pad, n + pad
    pa = _Pinned((m, lda), 7e9)
    pa.arr[:, :k] = a
    pc, pc2, po, pd = _Pinned((m, ldc)), _Pinned((m, n)), _Pinned((m, n)), _Pinned((m, nd))
    try:
        da = gu.dev(a)
        want = torch.empty((m, n), device="cuda")
        want2 = torch.empty((m, n), device="cuda")
        capi.matmul_multi([w, w2], da, m, [want, want2], stream=gu.stream())
        single = torch.empty((m, n), device="cuda")
        capi.matmul(w, da, m, single, stream=gu.stream())
        act = torch.empty((m, n), device="cuda")
        capi.mlp_swiglu(w, w2, da, m, act, stream=gu.stream())
        down = torch.empty((m, nd), device="cuda")
        capi.mlp_swiglu_down(w, w2, wd, da, m, down, stream=gu.stream())
        torch.cuda.synchronize()
        bits = lambda t: t.cpu().numpy().view(np.uint32)
        for _ in range(2):
            pc.arr[...] = -3.5
            pc.arr[:, :n] = np.nan
            capi.matmul(w, pa.addr, m, pc.addr, lda=lda, ldc=ldc, mem=capi.MEM_HOST)
            assert np.array_equal(pc.arr[:, :n].view(np.uint32), bits(single))
            assert np.all(pc.arr[:, n:] == np.float32(-3.5)), "the padding of the output rows was written"
            pc.arr[...] = np.nan
            pc2.arr[...] = np.nan
            capi.matmul_multi([w, w2], pa.addr, m, [pc.addr, pc2.addr], lda=lda, ldc=[ldc, n], mem=capi.MEM_HOST)
            assert np.array_equal(pc.arr[:, :n].view(np.uint32), bits(want))
            assert np.array_equal(pc2.arr.view(np.uint32), bits(want2))
            po.arr[...] = np.nan
            capi.mlp_swiglu(w, w2, pa.addr, m, po.addr, lda=lda, mem=capi.MEM_HOST)
            assert np.array_equal(po.arr.view(np.uint32), bits(act))
            pd.arr[...] = np.nan
            capi.mlp_swiglu_down(w, w2, wd, pa.addr, m, pd.addr, lda=lda, mem=capi.MEM_HOST)
            assert np.array_equal(pd.arr.view(np.uint32), bits(down))
    finally:
        for p in (pa, pc, pc2, po, pd):
            p.free()
        for x in (w, w2, wd):
            x.destroy()
