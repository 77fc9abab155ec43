"""GPU parity: activation quantizers must be bit-exact (int8 values, scales, group sums)
with the reference CPU quantizers, here restated by the oracle (and the reference
library itself when it is present)."""
import numpy as np
import pytest

from nntrainer_amd import synth

pytestmark = pytest.mark.gpu


def _cases(k):
    x = synth.normal(11, (64, k))
    x[0, :] = 0.0                      # all-zero blocks
    x[1, :k // 2] = 0.0                # partly zero
    x[2, 5] = 9.5; x[2, 9] = -9.5      # +amax before -amax
    x[3, 5] = -9.5; x[3, 9] = 9.5      # -amax before +amax
    x[4, :] *= 1e-6                    # tiny scale -> fp16 subnormal d for Q8_0
    x[5, :] *= 1e4                     # large scale
    x[6, 17] = 300.0                   # single spike
    x[7, :] = np.round(x[7, :] * 4) / 4  # many exact ties after scaling
    x[8, :] = 0.0; x[8, 100] = -1.0    # single non-zero, negative
    return x


@pytest.mark.parametrize("k", [256, 1024, 4096])
def test_q8_0_bit_exact(hipq, cr, k):
    import gpu_util as gu
    x = _cases(k)
    want = cr.quantize_act(cr.oracle(), "q8_0", x)
    got = gu.gpu_quantize("q8_0", x)
    assert got.shape == want.shape
    assert np.array_equal(got, want), "Q8_0 blocks differ in %d bytes" % (got != want).sum()
    if cr.ref() is not None:
        assert np.array_equal(got, cr.quantize_act(cr.ref(), "q8_0", x))


@pytest.mark.parametrize("variant", ["row", "mat"])
@pytest.mark.parametrize("k", [256, 2048, 4096])
def test_q8_K_bit_exact(hipq, cr, k, variant):
    import gpu_util as gu
    x = _cases(k)
    want = cr.quantize_act(cr.oracle(), "q8_K", x, variant)
    got = gu.gpu_quantize("q8_K", x, variant)
    assert np.array_equal(got, want), "Q8_K/%s blocks differ in %d bytes" % (variant, (got != want).sum())
    if cr.ref() is not None and variant == "row":
        assert np.array_equal(got, cr.quantize_act(cr.ref(), "q8_K", x, "row"))
    if cr.ref() is not None and variant == "mat":
        inter = np.stack([cr.interleave4("q8_K", got[4 * g:4 * g + 4], k) for g in range(x.shape[0] // 4)])
        assert np.array_equal(inter, cr.quantize_act(cr.ref(), "q8_K", x, "mat"))


def test_q8_K_rounding_adversaries(hipq, cr):
    """Inputs where rounding x*iscale once (row quantizer) and twice (4-row quantizer)
    give different integers: both variants must follow their own rule."""
    import gpu_util as gu
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "q8k_rounding_adversaries.npy")
    x = np.load(path).reshape(-1, 256)
    x = x[: (len(x) // 4) * 4]
    row = gu.gpu_quantize("q8_K", x, "row")
    mat = gu.gpu_quantize("q8_K", x, "mat")
    assert np.array_equal(row, cr.quantize_act(cr.oracle(), "q8_K", x, "row"))
    assert np.array_equal(mat, cr.quantize_act(cr.oracle(), "q8_K", x, "mat"))
    assert (row != mat).any()


def test_q8_large_full_size(hipq, cr):
    """Full prefill size (512 x 4096): every block bit-exact."""
    import gpu_util as gu
    x = synth.normal(1, (512, 4096))
    for kind, variant in (("q8_0", "row"), ("q8_K", "row"), ("q8_K", "mat")):
        want = cr.quantize_act(cr.oracle(), kind, x, variant)
        got = gu.gpu_quantize(kind, x, variant)
        assert np.array_equal(got, want), (kind, variant)


def _tiled_to_canonical(buf, m_rows, k):
    """Canonical (d, qs[256], pair sums[8]) per super-block out of the tiled form the Q4_K
    prefill product reads: rows tiled by 128; per 128-deep stage a 16 KB tile of 16-byte matrix
    operands [row / 32][step][lane group g * 32 + row % 32], an operand = the 8 even values of a
    16-value group, then its 8 odd ones; lane group g takes sub-blocks 4g .. 4g+3, two steps each."""
    nsb, mt_n = k // 256, (m_rows + 127) // 128
    mpad = mt_n * 128
    qt = buf[: mpad * k].view(np.int8)
    amin = buf[mpad * k: mpad * k + mpad * nsb * 32].view(np.float16)
    dat = buf[mpad * k + mpad * nsb * 32: mpad * k + mpad * nsb * 36].view(np.float32)
    d = np.zeros((mpad, nsb), np.float32)
    qs = np.zeros((mpad, nsb, 256), np.int8)
    lo6 = np.zeros((mpad, nsb, 8), np.float32)
    rest = np.zeros((mpad, nsb, 8), np.float32)
    for m in range(mpad):
        mt, r = m >> 7, m & 127
        for b in range(nsb):
            rb = (mt * nsb + b) * 128 + r
            d[m, b] = dat[rb]
            lo6[m, b] = amin[rb * 16: rb * 16 + 8]
            rest[m, b] = amin[rb * 16 + 8: rb * 16 + 16]
            for jb in range(8):
                for h in range(2):
                    g, st = jb >> 2, 2 * (jb & 3) + h
                    off = (mt * 2 * nsb + 2 * b + (st >> 2)) * 16384 + ((r >> 5) * 4 + (st & 3)) * 1024 \
                        + (g * 32 + (r & 31)) * 16
                    op = qt[off: off + 16]
                    v = np.empty(16, np.int8)
                    v[0::2], v[1::2] = op[:8], op[8:]
                    qs[m, b, jb * 32 + h * 16: jb * 32 + h * 16 + 16] = v
    return d, qs, lo6, rest


@pytest.mark.parametrize("m_rows,k", [(64, 256), (131, 768), (515, 1024), (30, 4096)])
def test_q8_K_tiled_form_matches_canonical(hipq, cr, m_rows, k):
    """The quantizer of the Q4_K prefill product (its own kernel: four rows per wavefront) holds
    the same values as the canonical blocks, which the tests above pin against the reference:
    rows below the last multiple of four follow the 4-row quantizer, the others the row one."""
    import torch
    import gpu_util as gu
    from nntrainer_amd import capi
    base = _cases(k)
    adv = np.load(__import__("os").path.join(__import__("os").path.dirname(__file__), "golden",
                                            "q8k_rounding_adversaries.npy")).reshape(-1, 256)
    x = synth.normal(5, (m_rows, k))
    n = min(m_rows, base.shape[0])
    x[:n] = base[:n]
    if m_rows > 70:  # adversarial super-blocks spread over rows of both kinds
        for i in range(min(len(adv), 48)):
            x[m_rows - 1 - i, (i % (k // 256)) * 256: (i % (k // 256)) * 256 + 256] = adv[i]
    x[m_rows - 1, :256] = 0.0
    x[m_rows - 2, 7] = 3.25; x[m_rows - 2, 200] = -3.25; x[m_rows - 2, :7] = 0.1
    mat = gu.gpu_quantize("q8_K", x, "mat").reshape(m_rows, k // 256, 292)
    row = gu.gpu_quantize("q8_K", x, "row").reshape(m_rows, k // 256, 292)
    mat_rows = (m_rows // 4) * 4
    want = np.concatenate([mat[:mat_rows], row[mat_rows:]])
    xd = torch.from_numpy(x).cuda()
    out = torch.zeros(capi.bench_tiled_bytes(m_rows, k), dtype=torch.uint8, device="cuda")
    capi.bench_quantize_tiled(xd, m_rows, k, out, stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    d, qs, lo6, rest = _tiled_to_canonical(out.cpu().numpy(), m_rows, k)
    want_d = want[:, :, :4].copy().view(np.float32)[:, :, 0]
    want_q = want[:, :, 4:260].view(np.int8)
    want_bs = want[:, :, 260:292].copy().view(np.int16).astype(np.int32)
    pair = want_bs[:, :, 0::2] + want_bs[:, :, 1::2]
    assert np.array_equal(d[:m_rows].view(np.uint32), want_d.view(np.uint32)), "scales differ"
    assert np.array_equal(qs[:m_rows], want_q), "%d int8 values differ" % (qs[:m_rows] != want_q).sum()
    assert np.array_equal(lo6[:m_rows], (pair & 63).astype(np.float32))
    assert np.array_equal(rest[:m_rows], (pair - (pair & 63)).astype(np.float32))
    # the padding rows of the last tile are zeros (the product reads them)
    assert not d[m_rows:].any() and not qs[m_rows:].any() and not lo6[m_rows:].any() and not rest[m_rows:].any()
