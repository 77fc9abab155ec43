"""Configuration C5: the quantized FC path inside a whole decoder.

Both legs run tests/c5_decoder.py; only the `fc` callable differs (CPU: the
reference library or the oracle; GPU: libhipq). Checked: every FC output of the
prefill step within the path's tolerance, and identical greedy token ids."""
import os

import numpy as np
import pytest

from nntrainer_amd import synth

pytestmark = pytest.mark.gpu

TOL = 1e-4  # max |gpu - cpu| / max |cpu| per FC output


def _run_both(cfg, cr, prompt_len, n_decode):
    import c5_decoder as c5
    weights, emb, used = c5.build_weights(cfg, cr)
    prompt = synth.token_ids(cfg.seed + 1000, prompt_len, cfg.vocab).tolist()
    cpu = c5.CpuFC(weights, cr)
    cpu_tokens, cpu_trace = c5.generate(cfg, emb, cpu, prompt, n_decode, trace_first=True)
    gpu = c5.GpuFC(weights)
    try:
        gpu_tokens, gpu_trace = c5.generate(cfg, emb, gpu, prompt, n_decode, trace_first=True)
    finally:
        gpu.close()
    return cpu_tokens, cpu_trace, gpu_tokens, gpu_trace


def _check(cpu_tokens, cpu_trace, gpu_tokens, gpu_trace):
    """Every FC of this model is Q4_0 (and the head one Q6_K row), whose products carry the reference's
    bits at every row count, and the two legs share everything else: the traced FC outputs of the
    prefill are equal bit for bit, not merely within the path's 1e-4."""
    assert len(cpu_trace) == len(gpu_trace)
    for (name, ref), (gname, got) in zip(cpu_trace, gpu_trace):
        assert name == gname
        err = float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))
        assert err <= TOL, (name, err)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (name, err)
    assert gpu_tokens == cpu_tokens, (gpu_tokens, cpu_tokens)


def test_small_decoder_prefill_and_decode(hipq, cr):
    import c5_decoder as c5
    cfg = c5.Config(layers=4, hidden=512, inter=1024, heads=8, kv_heads=4, head_dim=64, vocab=4096)
    _check(*_run_both(cfg, cr, prompt_len=48, n_decode=12))


@pytest.mark.skipif(os.environ.get("HIPQ_SKIP_FULL_C5") == "1", reason="full-size C5 disabled by HIPQ_SKIP_FULL_C5")
def test_c5_full_size(hipq, cr):
    """28 layers, hidden 1024, 512-token prompt, 128 greedy tokens."""
    import c5_decoder as c5
    cfg = c5.Config()
    cpu_tokens, cpu_trace, gpu_tokens, gpu_trace = _run_both(cfg, cr, prompt_len=512, n_decode=128)
    assert len(gpu_tokens) == 128
    _check(cpu_tokens, cpu_trace, gpu_tokens, gpu_trace)
