"""GPU parity: the offline weight quantizers emit the same bytes as the reference's
(restated by the oracle, which is itself pinned bit-for-bit to the reference library)."""
import numpy as np
import pytest

from nntrainer_amd import capi, synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["q4_0", "q4_K", "q6_K"])
@pytest.mark.parametrize("sigma", [0.02, 1.0])
def test_weight_quantizer_bytes(hipq, cr, kind, sigma):
    import gpu_util as gu
    import torch
    n, k = 512, 2048
    w = synth.normal(500, (n, k), sigma)
    w[3, :256] = 0.0
    w[5, 256:288] = 0.0
    w[7, 0:32] = 0.01
    want = cr.quantize_weights(cr.oracle(), kind, w)
    out = torch.zeros(capi.weight_nbytes(kind, n, k), dtype=torch.uint8, device="cuda")
    capi.quantize_weights(kind, gu.dev(w), n, k, out, stream=gu.stream())
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    nb = cr.BLOCK_BYTES[kind][0]
    bad = (got.reshape(-1, nb) != want.reshape(-1, nb)).any(1).sum()
    assert bad == 0, "%d of %d blocks differ" % (bad, got.size // nb)
