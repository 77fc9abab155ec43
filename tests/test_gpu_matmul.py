"""GPU parity: fp32 outputs of the quantized matmul (decode GEMV and prefill GEMM)
against the oracle on the same seeded inputs, through the C ABI.

Bar: max|gpu - ref| / max|ref| <= 1e-4 per matrix (only the order of the fp32
additions may differ; integer inner sums are exact on both sides)."""
import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu

KINDS = ["q4_0", "q4_K", "q6_K"]


def _weights(cr, kind, n, k, seed):
    w = synth.normal(seed, (n, k), 0.02)
    return cr.quantize_weights(cr.oracle(), kind, w)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n,k", [(256, 256), (512, 1024), (1000, 768), (4096, 4096), (768, 2048),
                                 (130, 8192), (64, 12288)])
def test_gemv_matches_oracle(hipq, cr, kind, n, k):
    import gpu_util as gu
    if kind != "q4_0" and k % 256:
        pytest.skip("K must be a multiple of 256")
    blocks = _weights(cr, kind, n, k, seed=100 + n)
    a = synth.normal(200 + k, (1, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
    # the decode path reproduces the reference's fp32 evaluation order: same bits
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n,k", [(6150, 4096), (8200, 4096), (12290, 4096), (2050, 3072), (1024, 3072),
                                 (3000, 2304), (2100, 2560), (9000, 2048), (33000, 4096), (33000, 2048),
                                 (1000, 1024), (40000, 1024)])
def test_single_row_against_the_instances_by_row_length(hipq, cr, kind, n, k):
    """One row against shapes chosen by what the library picks for them: the kernels with the row length as
    a constant (1024, 2048, 3072, 4096) and the ones that take any length (2304, 2560),
    workgroups of twelve wavefronts whose last one hangs over the matrix's end (6150, 12290), four wavefronts
    of four rows (8200), the plain and the streamed kernel behind the quantizer's launch (33000 and 40000
    columns). Same bits as the reference's row product."""
    import gpu_util as gu
    blocks = _weights(cr, kind, n, k, seed=900 + n % 97)
    a = synth.normal(950 + k % 89, (1, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert not np.isnan(got).any()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m", [2, 3, 4, 5, 7, 8])
def test_small_m_matches_oracle(hipq, cr, kind, m):
    """M = 2..8 runs the multi-row GEMV; rows below 4*(M/4) of a Q4_K matmul must be
    quantized with the 4-row rule, the rest with the row rule."""
    import gpu_util as gu
    n, k = 512, 1024
    blocks = _weights(cr, kind, n, k, seed=31)
    a = synth.normal(300 + m, (m, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m,n,k", [(3, 2304, 2048), (4, 2050, 4096), (5, 2056, 2048), (8, 4100, 2048),
                                   (7, 12288, 2048), (3, 8200, 1024), (4, 8195, 2048), (6, 1100, 768),
                                   (8, 1024, 256), (5, 3000, 4096), (8, 1030, 8192), (6, 1024, 5376),
                                   (4, 4100, 1280), (9, 1100, 1024), (14, 2048, 512), (16, 1024, 2048),
                                   (11, 4000, 4096), (6, 32768, 1024), (8, 8200, 4096), (24, 4096, 2048),
                                   (64, 2048, 2048), (33, 1056, 4096), (2, 16400, 1024), (4, 6150, 4096),
                                   (3, 12290, 4096), (4, 4100, 4096), (2, 33000, 2048)])
def test_small_m_on_large_matrices_matches_oracle(hipq, cr, kind, m, n, k):
    """Three to sixteen rows against larger matrices, where Q4_K leaves the GEMV engine (and, from
    nine rows, the prefill GEMM) for the matrix-core kernel of gemm_rows_q4k.hip (five rows and
    more from 1024 columns up, four from 4096 or, with rows of 4096, 6144, three from 8192 or 12288,
    two against 16384 rows of 1024; more than eight rows as passes
    of eight side by side in one launch, up to 64 rows where the product is small, the later
    passes with fewer rows under the 4-row rule or none): rows under the reference's
    4-row rule and under its row rule in one call
    (6 = 4 + 2), one to 32 super-blocks a row (a round of four wavefronts partly idle, a single
    round, rows longer than the GEMV engine's 4096-weight chunk), column counts that end inside
    a 32-column tile; five to eight rows against 2^25 weights and more, where Q4_0 takes its
    matrix-core GEMM. Same bits as the reference, for all three formats."""
    import gpu_util as gu
    blocks = _weights(cr, kind, n, k, seed=700 + n)
    a = synth.normal(701 + k + m, (m, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    engine_rows = 2 if n * k >= 2 ** 28 else 4 if n * k >= 2 ** 25 else 8 if n * k >= 2 ** 24 else 16
    if kind == "q6_K" and m > engine_rows:
        # Q6_K leaves the GEMV engine earlier on large matrices (the matrix cores are faster there)
        assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
        return
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("m,n,k", [(1, 65553, 1024), (1, 65536, 256), (2, 12300, 512), (3, 6150, 768),
                                   (2, 600, 1024), (3, 16000, 512), (4, 2050, 768), (2, 16500, 1024),
                                   (6, 1030, 1024), (8, 2048, 512), (5, 520, 768),
                                   (4, 6144, 1024), (5, 3100, 1280), (7, 3072, 256), (9, 640, 256),
                                   (12, 600, 2304), (16, 513, 1024), (17, 520, 5120), (40, 1500, 1024),
                                   (64, 4096, 256), (57, 2050, 1280)])
def test_q4_0_few_rows_on_the_matrix_cores_match_oracle(hipq, cr, m, n, k):
    """Q4_0 with a few rows where gemm_rows_q40.hip takes them (one row against a wide matrix of
    short rows, two rows from 12288 columns of 1024 or 32768 longer ones, three and four from 6144,
    two to eight from 512 where the kernel quantizes the rows itself, five to eight from 3072,
    nine to sixteen from 512, up to 64 while the launch stays small): one to eight passes, one to
    five rounds of 32 blocks with the last one partly or wholly one wavefront's, column counts
    that end inside a 32-column tile. Same bits as the reference."""
    import gpu_util as gu
    blocks = _weights(cr, "q4_0", n, k, seed=1300 + m)
    a = synth.normal(1301 + k + m, (m, k))
    ref = cr.gemm(cr.oracle(), "q4_0", a, blocks, n)
    w = capi.Weight("q4_0", n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n,k", [(32800, 1024), (33000, 512), (40010, 256), (32768, 768), (50000, 1280)])
def test_single_row_against_wide_matrices_of_short_rows(hipq, cr, kind, n, k):
    """One row against 32768 columns or more with rows of fewer than 64 load units: Q4_0 and Q4_K
    stream them sixteen lanes a row, eight rows a group and two or four groups a wavefront with the
    next group's loads in flight (Q6_K keeps the plain kernel); column counts that end inside a
    group and inside a workgroup's share. Same bits as the reference."""
    import gpu_util as gu
    blocks = _weights(cr, kind, n, k, seed=1600 + k)
    a = synth.normal(1601 + n, (1, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m,n,k", [(1, 8200, 12288), (3, 200, 8192), (8, 520, 9216), (1, 96, 20480),
                                   (5, 64, 4352)])
def test_rows_longer_than_one_chunk_match_oracle(hipq, cr, kind, m, n, k):
    """K above 4096 runs the GEMV instance that keeps the next chunk's weights in flight while
    the current chunk is computed: two, three and five chunks, a last chunk of 256, every group
    size the row count selects, one to eight activation rows. Same bits as the reference."""
    import gpu_util as gu
    blocks = _weights(cr, kind, n, k, seed=900 + n)
    a = synth.normal(901 + k + m, (m, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
        "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m,n,k", [(16, 256, 256), (64, 512, 1024), (130, 384, 512), (457, 512, 512),
                                   (459, 512, 512), (512, 1024, 2048)])
def test_gemm_matches_oracle(hipq, cr, kind, m, n, k):
    """Prefill shapes, including M % 4 != 0 (the reference's leftover-row path,
    unittest_nntrainer_cpu_backend.cpp:457-515 uses M = 457, 458, 459) and tiles that
    do not divide M or N."""
    import gpu_util as gu
    blocks = _weights(cr, kind, n, k, seed=41 + m)
    a = synth.normal(400 + m, (m, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
    if kind == "q4_0":
        # Q4_0 (one fma per 32-block, in block order) reproduces the reference's fp32 order:
        # same bits, so a decoder's prefill cannot drift from the CPU leg. The matrix-core
        # GEMMs of the K-formats (two int8 planes per product) do not claim that.
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
            "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)


@pytest.mark.parametrize("m,n,k", [(17, 128, 256), (33, 200, 768), (64, 96, 1024), (100, 1000, 512),
                                   (512, 4096, 4096), (1100, 8192, 512), (12, 8192, 4096)])
def test_q6_K_gemm_matches_oracle(hipq, cr, m, n, k):
    """The Q6_K prefill product on the matrix cores: one and three super-blocks per row,
    N not a multiple of the 32-row weight tiles or of the 128-column workgroup tiles, M not a
    multiple of the tile heights, a shape that takes the 128-row tiles, the size of a
    Q6_K FC of a 4096-wide model, and twelve rows against a matrix of 2^25 weights (from that
    size on more than four rows leave the GEMV engine). Four rows keep the GEMV engine and the
    reference's bits at every size here."""
    import gpu_util as gu
    blocks = _weights(cr, "q6_K", n, k, seed=61 + m)
    a = synth.normal(600 + m, (m, k))
    a[0, :] = 0.0                      # a row of zero scales
    a[m - 1, 3] = 40.0                 # a row whose scale is set by one value
    ref = cr.gemm(cr.oracle(), "q6_K", a, blocks, n)
    w = capi.Weight("q6_K", n, k, blocks)
    got = gu.gpu_matmul(w, a)
    again = gu.gpu_matmul(w, a)        # the weight's tile copy exists now
    few = gu.gpu_matmul(w, a[:4])
    w.destroy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
    assert np.array_equal(got, again)
    assert np.array_equal(few.view(np.uint32), ref[:4].view(np.uint32))
    # per row as well: a row of small outputs must not hide behind the matrix maximum
    scale = np.abs(ref).max(axis=1)
    rows = scale > 0
    assert (np.abs(got - ref).max(axis=1)[rows] / scale[rows]).max() <= gu.TOL


def test_gemm_random_shapes_all_formats(hipq, cr):
    """Prefill products at shapes drawn from a seeded generator: N from 1 upward (narrower than a
    weight tile, between tile sizes), M between the GEMV limit and a few tiles, K one to five
    super-blocks. Every kernel's edge handling (padding rows and columns, odd super-block counts,
    both tile heights) is on some draw; the bar is the one of the fixed shapes."""
    import gpu_util as gu
    rng = np.random.RandomState(20240611)
    for case in range(24):
        kind = KINDS[case % 3]
        m = int(rng.choice([9, 17, 31, 64, 65, 127, 130, 257, 300]))
        n = int(rng.choice([1, 7, 31, 33, 100, 128, 129, 640, 1000, 4100]))
        k = 256 * int(rng.randint(1, 6))
        blocks = _weights(cr, kind, n, k, seed=500 + case)
        a = synth.normal(700 + case, (m, k))
        ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
        w = capi.Weight(kind, n, k, blocks)
        got = gu.gpu_matmul(w, a)
        w.destroy()
        assert not np.isnan(got).any(), (kind, m, n, k)
        assert gu.rel_err(got, ref) <= gu.TOL, (kind, m, n, k, gu.rel_err(got, ref))
        if kind == "q4_0":
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (kind, m, n, k)


@pytest.mark.parametrize("kind", ["q4_K", "q6_K"])
@pytest.mark.parametrize("m,n,k", [(17, 512, 2048), (40, 1000, 2304), (64, 4100, 4096), (100, 640, 3072),
                                   (128, 1536, 2048), (33, 1001, 2048)])
def test_k_format_gemm_in_parts_of_k(hipq, cr, kind, m, n, k):
    """Few tiles (up to 128 rows against a few thousand columns): once the weight has its tile copy
    the Q4_K and Q6_K prefill products are formed in parts of K that run side by side and are added in
    ascending order (nine super-blocks split 5 + 4, sixteen into four and eight parts). The first
    call, which makes the copy, and the following ones have the same bits, within 1e-4 of the
    reference; a strided output keeps its padding; N not a multiple of four takes no parts."""
    import gpu_util as gu
    import torch
    blocks = _weights(cr, kind, n, k, seed=330 + m)
    a = synth.normal(331 + m, (m, k))
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    w = capi.Weight(kind, n, k, blocks)
    try:
        first = gu.gpu_matmul(w, a)
        assert gu.rel_err(first, ref) <= gu.TOL, gu.rel_err(first, ref)
        ldc = n + 12
        dc = torch.full((m, ldc), float("nan"), device="cuda")
        capi.matmul(w, gu.dev(a), m, dc, ldc=ldc, stream=gu.stream())
        torch.cuda.synchronize()
        got = dc[:, :n].cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)
        assert torch.isnan(dc[:, n:]).all(), "the call wrote between the rows of C"
        assert np.array_equal(got, first), "the first call differs from the second"
        scale = np.abs(ref).max(axis=1)
        assert (np.abs(got - ref).max(axis=1) / scale).max() <= gu.TOL
        again = torch.full((m, n), float("nan"), device="cuda")
        capi.matmul_noalloc(w, gu.dev(a), m, again, stream=gu.stream())
        torch.cuda.synchronize()
        assert np.array_equal(again.cpu().numpy(), got), "the allocation-free call differs"
    finally:
        w.destroy()


def test_q4_K_gemm_tall_tiles(hipq, cr):
    """A shape for which the Q4_K GEMM picks its 128-row tiles (two rounds of 64-row
    tiles against one of 128-row tiles), with M not a multiple of the tile height."""
    import gpu_util as gu
    m, n, k = 1000, 8192, 512
    blocks = _weights(cr, "q4_K", n, k, seed=47)
    a = synth.normal(447, (m, k))
    ref = cr.gemm(cr.oracle(), "q4_K", a, blocks, n)
    w = capi.Weight("q4_K", n, k, blocks)
    got = gu.gpu_matmul(w, a)
    w.destroy()
    assert not np.isnan(got).any()
    assert gu.rel_err(got, ref) <= gu.TOL, gu.rel_err(got, ref)


@pytest.mark.parametrize("kind", ["q4_0", "q4_K"])
def test_x8_layout_equals_canonical(hipq, cr, kind):
    """Weights handed over in NNTrainer's 8-row interleave give the same outputs."""
    import gpu_util as gu
    n, k = 512, 1024
    blocks = _weights(cr, kind, n, k, seed=51)
    x8 = cr.repack_x8(cr.oracle(), kind, blocks, n, k)
    a = synth.normal(52, (5, k))
    w0 = capi.Weight(kind, n, k, blocks)
    w1 = capi.Weight(kind, n, k, x8, layout=capi.LAYOUT_X8)
    c0, c1 = gu.gpu_matmul(w0, a), gu.gpu_matmul(w1, a)
    w0.destroy(); w1.destroy()
    assert np.array_equal(c0, c1)


def test_host_memory_entry(hipq, cr):
    """HIPQ_MEM_HOST: plain host pointers in and out, with row strides."""
    import gpu_util as gu
    n, k, m = 256, 512, 3
    blocks = _weights(cr, "q4_K", n, k, seed=61)
    a = np.zeros((m, k + 64), np.float32)
    a[:, :k] = synth.normal(62, (m, k))
    c = np.full((m, n + 16), np.nan, np.float32)
    w = capi.Weight("q4_K", n, k, blocks)
    capi.matmul(w, a, m, c, lda=k + 64, ldc=n + 16, mem=capi.MEM_HOST)
    w.destroy()
    ref = cr.gemm(cr.oracle(), "q4_K", a[:, :k], blocks, n)
    assert gu.rel_err(c[:, :n], ref) <= gu.TOL
    assert np.isnan(c[:, n:]).all()


def test_matmul_multi_shares_quantization(hipq, cr):
    import gpu_util as gu
    import torch
    k, m = 1024, 1
    ns = [512, 256, 256]
    blocks = [_weights(cr, "q4_0", n, k, seed=70 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight("q4_0", n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(73, (m, k))
    da = gu.dev(a)
    outs = [torch.empty((m, n), device="cuda") for n in ns]
    capi.matmul_multi(ws, da, m, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for n, b, o in zip(ns, blocks, outs):
        assert gu.rel_err(o.cpu().numpy(), cr.gemm(cr.oracle(), "q4_0", a, b, n)) <= gu.TOL
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n,k", [(8, 256), (37, 256), (1000, 768), (1024, 1024), (3072, 1024), (2050, 2048),
                                 (4096, 4096), (8200, 3072), (12288, 4096)])
def test_decode_row_quantized_in_the_gemv_equals_the_two_launches(hipq, cr, kind, n, k):
    """hipq_matmul with one row on a small matrix runs one kernel whose workgroups
    quantize the row themselves; the multi-weight entry with more than four weights
    keeps the quantizer kernel and the GEMV on its blocks. Same arithmetic, so the
    outputs are the same bits; the oracle pins both."""
    import gpu_util as gu
    import torch
    blocks = _weights(cr, kind, n, k, seed=500 + n)
    a = synth.normal(600 + k, (1, k))
    a[0, 5] = 0.0
    if k >= 512:
        a[0, 256:512] = 0.0   # an all-zero block: scale 0
    w = capi.Weight(kind, n, k, blocks)
    one = gu.gpu_matmul(w, a)
    two = [torch.full((1, n), float("nan"), device="cuda") for _ in range(5)]
    capi.matmul_multi([w] * 5, gu.dev(a), 1, two, stream=gu.stream())
    torch.cuda.synchronize()
    w.destroy()
    for t in two:
        assert np.array_equal(one, t.cpu().numpy())
    ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
    assert gu.rel_err(one, ref) <= gu.TOL


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("k,ns", [(1024, [2048, 1024, 1024]), (1024, [3072, 3072]), (256, [8, 37, 4, 130]),
                                  (4096, [4096]), (2048, [1000, 6150])])
def test_decode_row_on_several_weights_is_one_launch_with_the_same_bits(hipq, cr, kind, k, ns):
    """Up to four weights of one format and K on one row go out as a single launch
    (Q, K and V, or gate and up, of a decoder layer); the outputs are those of
    hipq_matmul on each weight."""
    import gpu_util as gu
    import torch
    blocks = [_weights(cr, kind, n, k, seed=700 + n + i) for i, n in enumerate(ns)]
    ws = [capi.Weight(kind, n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(710 + k, (1, k))
    outs = [torch.full((1, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), 1, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for w, b, n, o in zip(ws, blocks, ns, outs):
        assert np.array_equal(o.cpu().numpy(), gu.gpu_matmul(w, a))
        assert gu.rel_err(o.cpu().numpy(), cr.gemm(cr.oracle(), kind, a, b, n)) <= gu.TOL
    for w in ws:
        w.destroy()


def test_decode_calls_replay_from_a_captured_graph(hipq, cr):
    """The one-row calls are single kernel launches without allocations, so a caller
    can capture a decoder layer's FCs in a graph. Every replay, with other work on
    the device in between, gives the bits of the direct calls."""
    import gpu_util as gu
    import torch
    k, ns = 1024, [2048, 1024, 1024]
    blocks = [_weights(cr, "q4_0", n, k, seed=800 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight("q4_0", n, k, b) for n, b in zip(ns, blocks)]
    wo = capi.Weight("q4_0", k, 2048, _weights(cr, "q4_0", k, 2048, seed=810))
    x = torch.zeros((1, k), device="cuda")
    qkv = [torch.zeros((1, n), device="cuda") for n in ns]
    y = torch.zeros((1, k), device="cuda")

    def layer(stream):
        capi.matmul_multi(ws, x, 1, qkv, stream=stream)
        capi.matmul(wo, qkv[0], 1, y, stream=stream)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(side.cuda_stream)          # first calls outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer(side.cuda_stream)
    for it in range(4):
        x.copy_(gu.dev(synth.normal(820 + it, (1, k))))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in qkv] + [y.clone()]
        scratch = torch.randn(1 << 20, device="cuda").sum()   # other work between the replays
        layer(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for g, e in zip(got, qkv + [y]):
            assert torch.equal(g, e), "replay %d differs from the direct calls" % it
        assert torch.isfinite(scratch)
    for w in ws + [wo]:
        w.destroy()


@pytest.mark.parametrize("own_streams", [False, True])
def test_calls_from_several_threads(hipq, cr, own_streams):
    """The entry points are called from several threads (the reference's expert loop
    runs Tensor::dot inside an OpenMP loop, qwen_moe_layer.cpp:478-490; model load uses a
    thread per node). Calls that name the same stream share its scratch: their launches
    must not interleave. Every result equals the one a single thread gets."""
    import threading
    import gpu_util as gu
    import torch
    n, k = 384, 512
    ws = {kind: capi.Weight(kind, n, k, _weights(cr, kind, n, k, seed=950)) for kind in ("q4_0", "q4_K")}
    cases = [(kind, m) for kind in ws for m in (1, 5, 40)]
    acts = {m: gu.dev(synth.normal(960 + m, (m, k))) for m in (1, 5, 40)}
    want = {}
    for kind, m in cases:
        c = torch.empty((m, n), device="cuda")
        capi.matmul(ws[kind], acts[m], m, c, stream=gu.stream())
        torch.cuda.synchronize()
        want[(kind, m)] = c.clone()
    errors = []

    def work(tid):
        try:
            st = torch.cuda.Stream() if own_streams else torch.cuda.current_stream()
            outs = {cs: torch.empty((cs[1], n), device="cuda") for cs in cases}
            for it in range(25):
                for kind, m in cases[tid % 2:] + cases[:tid % 2]:
                    capi.matmul(ws[kind], acts[m], m, outs[(kind, m)], stream=st.cuda_stream)
                st.synchronize()
                for cs in cases:
                    if not torch.equal(outs[cs], want[cs]):
                        errors.append((tid, it, cs))
                        return
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for w in ws.values():
        w.destroy()
    assert not errors, errors[:3]


def test_weights_read_from_a_model_file(hipq, cr, tmp_path):
    """A file laid out as NNTrainer writes MODEL_FORMAT_BIN (tensors back to back, Q4_0 and
    Q4_K in the 8-row interleave, a scheme word in front of Q4_K only): the handles read
    from it multiply like handles made from the same bytes."""
    import gpu_util as gu
    specs = [("q4_0", 512, 1024), ("q4_K", 256, 512), ("q6_K", 384, 256), ("q4_K", 128, 256)]
    blocks = [_weights(cr, kind, n, k, seed=900 + i) for i, (kind, n, k) in enumerate(specs)]
    stored = [cr.repack_x8(cr.oracle(), kind, b, n, k) if kind != "q6_K" else b
              for (kind, n, k), b in zip(specs, blocks)]
    path = tmp_path / "model.bin"
    listing = [("skip", 4096)]
    with open(path, "wb") as f:
        f.write(b"\0" * 7)                            # the caller's start offset
        f.write(np.arange(1024, dtype=np.float32).tobytes())
        for (kind, n, k), b in zip(specs, stored):
            if kind == "q4_K":
                f.write(np.uint16(3).tobytes())       # QScheme::Q4_Kx8
            f.write(np.ascontiguousarray(b).tobytes())
            listing.append((kind, n, k, capi.LAYOUT_X8 if kind != "q6_K" else capi.LAYOUT_CANONICAL))
        f.write(b"tail")
    ws, end = capi.weights_from_file(path, listing, offset=7)
    assert ws[0] is None and end == path.stat().st_size - 4
    for w, (kind, n, k), b in zip(ws[1:], specs, blocks):
        a = synth.normal(910 + n, (3, k))
        ref = capi.Weight(kind, n, k, b)
        assert np.array_equal(gu.gpu_matmul(w, a), gu.gpu_matmul(ref, a))
        ref.destroy()
        w.destroy()
    # a Q4_Kx8 tensor listed as canonical, and a file that ends early, leave no handle behind
    with pytest.raises(capi.HipqError):
        capi.weights_from_file(path, [("skip", 4096), ("q4_0", 512, 1024, capi.LAYOUT_X8), ("q4_K", 256, 512)],
                               offset=7)
    with pytest.raises(capi.HipqError):
        capi.weights_from_file(path, listing + [("q6_K", 4096, 4096)], offset=7)


@pytest.mark.parametrize("kind,m", [("q4_K", 1), ("q4_K", 40), ("q6_K", 3), ("q6_K", 40)])
def test_matmul_multi_other_formats_and_prefill(hipq, cr, kind, m):
    """The multi-weight entry with the Q8_K formats, one row and a prefill chunk (the
    Q4_K prefill goes through the tiled activations and the matrix-core GEMM)."""
    import gpu_util as gu
    import torch
    k = 512
    ns = [384, 128, 256]
    blocks = [_weights(cr, kind, n, k, seed=80 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight(kind, n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(83, (m, k))
    outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), m, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for n, b, o in zip(ns, blocks, outs):
        got = o.cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, cr.gemm(cr.oracle(), kind, a, b, n)) <= gu.TOL
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("m", [4, 6])
def test_matmul_multi_few_rows_mixed_paths(hipq, cr, m):
    """A few rows against Q4_K weights of different sizes (and a Q6_K one) in one multi-weight call:
    the large Q4_K matrices take the matrix-core kernel (one quantization in its row form shared by
    them), the small one and the Q6_K one the GEMV engine with their own quantizations. All carry
    the reference's bits, whatever the order of the weights in the call."""
    import gpu_util as gu
    import torch
    k = 1024
    kinds, ns = ["q4_K", "q4_K", "q6_K", "q4_K", "q4_K"], [8192, 512, 640, 1056, 8200]
    blocks = [_weights(cr, kd, n, k, seed=95 + i) for i, (kd, n) in enumerate(zip(kinds, ns))]
    ws = [capi.Weight(kd, n, k, b) for kd, n, b in zip(kinds, ns, blocks)]
    a = synth.normal(99 + m, (m, k))
    outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), m, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for kd, n, b, o in zip(kinds, ns, blocks, outs):
        ref = cr.gemm(cr.oracle(), kd, a, b, n)
        assert np.array_equal(o.cpu().numpy().view(np.uint32), ref.view(np.uint32)), (kd, n)
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("k", [4096, 3072, 2304, 1024])
def test_matmul_multi_one_row_one_launch_by_row_length(hipq, cr, kind, k):
    """One row against the Q, K, V of a layer (one launch that quantizes the row itself): the launch with the
    row length as a constant (4096, 3072, 1024) and for any length (2304), widths that end inside a
    wavefront's group of rows. Every output carries the reference's bits."""
    import gpu_util as gu
    import torch
    ns = [4100, 1024, 1030] if k >= 3072 else [2050, 520, 512]
    blocks = [_weights(cr, kind, n, k, seed=1450 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight(kind, n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(1460 + k % 13, (1, k))
    outs = [torch.full((1, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), 1, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for n, b, o in zip(ns, blocks, outs):
        got = o.cpu().numpy()
        ref = cr.gemm(cr.oracle(), kind, a, b, n)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (n, gu.rel_err(got, ref))
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("m,k", [(2, 1024), (8, 1280), (13, 256), (16, 2048), (40, 1024), (64, 512)])
def test_matmul_multi_q4_0_few_rows_one_launch(hipq, cr, m, k):
    """A few rows against several Q4_0 weights of one K (Q, K, V or gate, up of a decode step of a
    batch): the weights' column tiles side by side in one launch of the few-rows kernel, four
    weights a launch (five make a launch of four and a single product), widths that end inside a
    32-column tile, outputs with a row stride. Every output carries the reference's bits."""
    import gpu_util as gu
    import torch
    ns = [2048, 1000, 1024, 72, 520]
    blocks = [_weights(cr, "q4_0", n, k, seed=1400 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight("q4_0", n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(1410 + m, (m, k))
    outs = [torch.full((m, n + 8 * i), float("nan"), device="cuda") for i, n in enumerate(ns)]
    capi.matmul_multi(ws, gu.dev(a), m, outs, ldc=[n + 8 * i for i, n in enumerate(ns)], stream=gu.stream())
    torch.cuda.synchronize()
    for i, (n, b, o) in enumerate(zip(ns, blocks, outs)):
        got = o.cpu().numpy()
        ref = cr.gemm(cr.oracle(), "q4_0", a, b, n)
        assert np.array_equal(got[:, :n].view(np.uint32), ref.view(np.uint32)), (n, gu.rel_err(got[:, :n], ref))
        assert np.isnan(got[:, n:]).all(), "the call wrote between the rows of an output"
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("m,k", [(2, 1024), (3, 512), (6, 1280), (13, 256), (16, 2048), (40, 1024)])
def test_matmul_multi_q4_K_few_rows_one_launch(hipq, cr, m, k):
    """The same for Q4_K weights: one quantization in the row form of the matrix-core kernels (rows
    below 4 * (m / 4) under the 4-row rule), then the weights' column tiles side by side in one launch
    of gemm_rows_q4k.hip, four weights a launch. The reference's bits for every output, and the bits
    of the single-weight call where that one keeps them (the single call of a wide weight with more
    than 16 rows takes the prefill GEMM, which agrees to 1e-4)."""
    import gpu_util as gu
    import torch
    ns = [2048, 1000, 1024, 72, 520]
    blocks = [_weights(cr, "q4_K", n, k, seed=1500 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight("q4_K", n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(1510 + m, (m, k))
    a[1, 3] = 8.5
    a[1, 7] = -8.5
    outs = [torch.full((m, n + 8 * i), float("nan"), device="cuda") for i, n in enumerate(ns)]
    capi.matmul_multi(ws, gu.dev(a), m, outs, ldc=[n + 8 * i for i, n in enumerate(ns)], stream=gu.stream())
    torch.cuda.synchronize()
    for i, (n, b, o) in enumerate(zip(ns, blocks, outs)):
        got = o.cpu().numpy()
        ref = cr.gemm(cr.oracle(), "q4_K", a, b, n)
        assert np.array_equal(got[:, :n].view(np.uint32), ref.view(np.uint32)), (n, gu.rel_err(got[:, :n], ref))
        assert np.isnan(got[:, n:]).all(), "the call wrote between the rows of an output"
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("ns", [[72, 3072], [3072, 72, 1000]])
def test_matmul_multi_q6_K_members_of_different_size_share_the_quantization(hipq, cr, ns):
    """Q6_K weights of one multi-weight call share the quantized rows of the first one's product. A
    product of few tiles keeps its partial products of parts of K behind those rows in the same
    workspace, and a later, larger member needs more of it: the workspace is sized for the largest
    member before the first product, so that it does not move between them. A fresh stream, so that
    the workspace starts empty."""
    import gpu_util as gu
    import torch
    m, k = 65, 2048
    blocks = [_weights(cr, "q6_K", n, k, seed=1700 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight("q6_K", n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(1710, (m, k))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        da = gu.dev(a)
        outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
        side.synchronize()
        capi.matmul_multi(ws, da, m, outs, stream=side.cuda_stream)
        side.synchronize()
    for n, b, o in zip(ns, blocks, outs):
        got = o.cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, cr.gemm(cr.oracle(), "q6_K", a, b, n)) <= gu.TOL, n
    for w in ws:
        w.destroy()


def test_matmul_multi_seeded_mixed_calls(hipq, cr):
    """Forty multi-weight calls drawn from a seeded generator: one to seven weights of mixed formats
    and widths, one to 130 rows, every second call on a stream of its own (an empty workspace).
    Whatever grouping the call chooses (one launch for several weights, shared quantizations, parts
    of K), every output is within 1e-4 of the reference and Q4_0 outputs carry its bits."""
    import gpu_util as gu
    import torch
    rng = np.random.default_rng(7)
    cache = {}

    def blocks_of(kind, n, k):
        if (kind, n, k) not in cache:
            cache[(kind, n, k)] = _weights(cr, kind, n, k, seed=2000 + n + k + len(kind))
        return cache[(kind, n, k)]

    for it in range(40):
        k = int(rng.choice([256, 512, 1024, 1280, 2048]))
        cnt = int(rng.integers(1, 8))
        kinds = [str(rng.choice(["q4_0", "q4_0", "q4_K", "q4_K", "q6_K"])) for _ in range(cnt)]
        ns = [int(rng.choice([72, 256, 520, 1000, 1024, 2048, 3072, 4100])) for _ in range(cnt)]
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 13, 16, 17, 31, 40, 64, 65, 130]))
        a = synth.normal(3000 + it, (m, k))
        if m > 1:
            a[1, 3] = 7.5
            a[1, 9] = -7.5
        blocks = [blocks_of(kd, n, k) for kd, n in zip(kinds, ns)]
        ws = [capi.Weight(kd, n, k, b) for kd, n, b in zip(kinds, ns, blocks)]
        outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
        da = gu.dev(a)
        st = torch.cuda.Stream() if it % 2 else torch.cuda.current_stream()
        torch.cuda.synchronize()
        capi.matmul_multi(ws, da, m, outs, stream=st.cuda_stream)
        torch.cuda.synchronize()
        for kd, n, b, o in zip(kinds, ns, blocks, outs):
            got = o.cpu().numpy()
            ref = cr.gemm(cr.oracle(), kd, a, b, n)
            case = (it, m, k, kd, n)
            assert not np.isnan(got).any(), case
            assert gu.rel_err(got, ref) <= gu.TOL, case
            if kd == "q4_0":
                assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), case
        for w in ws:
            w.destroy()


def test_matmul_multi_mixed_k_formats_prefill(hipq, cr):
    """Q4_K and Q6_K weights in one multi-weight prefill call: both take tiled Q8_K activations, but
    the reference quantizes the rows of a Q4_K product four at a time and those of a Q6_K product one
    by one (different sign rules), so the two groups must not share one quantization. Row 2 holds
    +amax before -amax, where the two quantizers differ."""
    import gpu_util as gu
    import torch
    m, k = 40, 512
    kinds, ns = ["q4_K", "q6_K", "q4_K", "q6_K"], [256, 160, 128, 384]
    blocks = [_weights(cr, kd, n, k, seed=90 + i) for i, (kd, n) in enumerate(zip(kinds, ns))]
    ws = [capi.Weight(kd, n, k, b) for kd, n, b in zip(kinds, ns, blocks)]
    a = synth.normal(93, (m, k))
    a[2, 5] = 9.5
    a[2, 9] = -9.5
    outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), m, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for kd, n, b, o, w in zip(kinds, ns, blocks, outs, ws):
        got = o.cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, cr.gemm(cr.oracle(), kd, a, b, n)) <= gu.TOL
        assert np.array_equal(got, gu.gpu_matmul(w, a)), "the multi-weight call differs from the single one"
    for w in ws:
        w.destroy()


@pytest.mark.parametrize("kind", ["q4_K", "q4_0"])
def test_matmul_multi_prefill_five_weights_one_launch_per_four(hipq, cr, kind):
    """Prefill products of several weights go out up to four a launch (column tiles of the weights
    side by side in one grid): five weights make a launch of four and one of one; widths that are
    no multiple of the workgroup's column tile; every output equals the single-weight call's."""
    import gpu_util as gu
    import torch
    m, k = 300, 1024
    ns = [512, 96, 200, 1024, 136]
    blocks = [_weights(cr, kind, n, k, seed=110 + i) for i, n in enumerate(ns)]
    ws = [capi.Weight(kind, n, k, b) for n, b in zip(ns, blocks)]
    a = synth.normal(113, (m, k))
    outs = [torch.full((m, n), float("nan"), device="cuda") for n in ns]
    capi.matmul_multi(ws, gu.dev(a), m, outs, stream=gu.stream())
    torch.cuda.synchronize()
    for n, b, o, w in zip(ns, blocks, outs, ws):
        got = o.cpu().numpy()
        assert not np.isnan(got).any()
        assert gu.rel_err(got, cr.gemm(cr.oracle(), kind, a, b, n)) <= gu.TOL
        assert np.array_equal(got, gu.gpu_matmul(w, a)), "the multi-weight call differs from the single one"
    for w in ws:
        w.destroy()


def test_bad_arguments_are_reported(hipq):
    with pytest.raises(capi.HipqError) as e:
        capi.weight_nbytes("q4_K", 16, 100)  # K not a multiple of 256 (q4_k_tensor.cpp:23-27)
    assert e.value.code == -1
    blocks = np.zeros(capi.weight_nbytes("q6_K", 8, 256), np.uint8)
    with pytest.raises(capi.HipqError):
        capi.Weight("q6_K", 8, 256, blocks, layout=capi.LAYOUT_X8)  # no x8 form of Q6_K
    blocks = np.zeros(capi.weight_nbytes("q4_0", 12, 64), np.uint8)
    with pytest.raises(capi.HipqError):
        capi.Weight("q4_0", 12, 64, blocks, layout=capi.LAYOUT_X8)  # N % 8 != 0 (repack returns -1)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("rows,n,k", [(8, 1100, 1024), (5, 512, 768), (12, 2048, 512), (16, 300, 256),
                                      (37, 1056, 1024), (3, 8200, 512), (1, 640, 256), (70, 1030, 512)])
def test_matmul_each_row_has_the_bits_of_single_row_products(hipq, cr, kind, rows, n, k):
    """hipq_matmul_each_row: the rows of a batch of decode steps against one weight in one call, every
    row with the bits of its own M = 1 product (the reference's loop over batch entries). For Q4_K
    that differs from hipq_matmul with M = rows (no 4-row quantizer, no pairwise sums): row 1 holds
    +amax before -amax, where the two quantizers round differently. Large and small matrices (the
    matrix-core kernel and the GEMV engine), more than 16 rows (several steps), strided rows, and
    host memory."""
    import gpu_util as gu
    import torch
    blocks = _weights(cr, kind, n, k, seed=500 + n)
    a = synth.normal(501 + rows + k, (rows, k))
    if rows > 1:
        a[1, 3] = 7.25
        a[1, 11] = -7.25
    ref = np.concatenate([cr.gemm(cr.oracle(), kind, a[r:r + 1], blocks, n) for r in range(rows)], axis=0)
    w = capi.Weight(kind, n, k, blocks)
    try:
        lda, ldc = k + 64, n + 32
        da = torch.zeros((rows, lda), device="cuda")
        da[:, :k] = gu.dev(a)
        dc = torch.full((rows, ldc), float("nan"), device="cuda")
        capi.matmul_each_row(w, da, rows, dc, lda=lda, ldc=ldc, stream=gu.stream())
        torch.cuda.synchronize()
        got = dc[:, :n].cpu().numpy()
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), \
            "%d of %d outputs differ in bits" % ((got.view(np.uint32) != ref.view(np.uint32)).sum(), got.size)
        assert torch.isnan(dc[:, n:]).all(), "the call wrote between the rows of C"
        host = np.full((rows, n), np.nan, np.float32)
        capi.matmul_each_row(w, a, rows, host, mem=capi.MEM_HOST, stream=gu.stream())
        assert np.array_equal(host.view(np.uint32), ref.view(np.uint32))
        single = gu.gpu_matmul(w, a[1:2]) if rows > 1 else None
        if single is not None:
            assert np.array_equal(single.view(np.uint32), ref[1:2].view(np.uint32))
    finally:
        w.destroy()


def test_row_counts_across_the_kernel_choices(hipq, cr):
    """hipq_matmul picks among the GEMV engine, the few-rows matrix-core kernel (one to eight passes),
    the prefill GEMMs (whole K or parts of K) by format, row count and matrix size. Shapes drawn
    around the thresholds from a seeded generator: every result within 1e-4 of the reference, Q4_0
    and every product of one or two rows with its bits, a second call the bits of the first."""
    import gpu_util as gu
    rng = np.random.RandomState(20250117)
    done = 0
    while done < 36:
        kind = KINDS[done % 3]
        n = int(rng.choice([1000, 1024, 1056, 2048, 4096, 4100, 8192, 8200]))
        k = int(rng.choice([256, 1024, 2048, 2304, 4096]))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 12, 16, 17, 24, 33, 48, 64, 65, 70]))
        if m * n * k > 4e8:
            continue
        blocks = _weights(cr, kind, n, k, seed=1200 + done)
        a = synth.normal(1300 + done, (m, k))
        ref = cr.gemm(cr.oracle(), kind, a, blocks, n)
        w = capi.Weight(kind, n, k, blocks)
        got = gu.gpu_matmul(w, a)
        again = gu.gpu_matmul(w, a)
        w.destroy()
        case = (kind, m, n, k)
        assert not np.isnan(got).any(), case
        assert gu.rel_err(got, ref) <= gu.TOL, (case, gu.rel_err(got, ref))
        assert np.array_equal(got, again), case
        if kind == "q4_0" or m <= 2:
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), case
        done += 1

