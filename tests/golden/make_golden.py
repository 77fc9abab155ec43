"""Regenerates the fixtures in this directory.

 oracle_digests.json        sha256 prefixes of oracle outputs on seeded inputs. Only written
                            when the reference library (oracle/_ref, compiled from the
                            reference's own sources) is present and agrees bit-for-bit with
                            the oracle on every case, so the digests are the reference's.
 q8k_rounding_adversaries.npy  256-value blocks on which rounding x*iscale once (fused
                            multiply-add, the row quantizer) and twice (rounded product, the
                            4-row quantizer) give different integers; found by search with
                            numpy only.
Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))


def rounding_adversaries(want=24):
    rng = np.random.default_rng(1)
    found = []
    while sum(len(f) for f in found) < want:
        xb = rng.standard_normal((65536, 256)).astype(np.float32)
        idx = np.abs(xb).argmax(1)
        mx = xb[np.arange(len(xb)), idx]
        iscale = (np.float32(-127.0) / mx).astype(np.float32)
        once = (iscale[:, None].astype(np.float64) * xb.astype(np.float64) + 12582912.0).astype(np.float32)
        twice = ((iscale[:, None] * xb).astype(np.float32) + np.float32(12582912.0)).astype(np.float32)
        hit = (once != twice).any(1)
        if hit.any():
            found.append(xb[hit])
    return np.concatenate(found)[:want + 1]


def main():
    import cpuref as cr
    import test_oracle_pinned as t

    adv = os.path.join(HERE, "q8k_rounding_adversaries.npy")
    if not os.path.exists(adv):
        np.save(adv, rounding_adversaries())
    if cr.ref() is None:
        sys.exit("reference library not built: digests are only written where it can vouch for them")
    # every digested output is first compared with the reference itself
    o, r = cr.oracle(), cr.ref()
    from nntrainer_amd import synth
    for kind in t.KINDS:
        w = t._w(20, 64, 1024)
        q = cr.quantize_weights(o, kind, w)
        assert np.array_equal(q, cr.quantize_weights(r, kind, w)), kind
        for m in (1, 6):
            a = synth.normal(21 + m, (m, 1024))
            assert np.array_equal(cr.gemm(o, kind, a, q, 64).view(np.uint32), cr.gemm(r, kind, a, q, 64).view(np.uint32))
    x = t._act_cases(1024)
    for kind in ("q8_0", "q8_K"):
        assert np.array_equal(cr.quantize_act(o, kind, x, "row"), cr.quantize_act(r, kind, x, "row"))
        mo = cr.quantize_act(o, kind, x, "mat")
        inter = np.stack([cr.interleave4(kind, mo[4 * g:4 * g + 4], 1024) for g in range(len(x) // 4)])
        assert np.array_equal(inter, cr.quantize_act(r, kind, x, "mat"))
    ys, zs = t._swiglu_inputs()
    for alpha in (None, 1.702):
        assert np.array_equal(cr.swiglu_x86(o, ys, zs, alpha).view(np.uint32), cr.swiglu_x86(r, ys, zs, alpha).view(np.uint32))
    # the cached mixture-of-experts oracle against the same block composed from the reference's routines
    for gpt_oss in (False, True):
        t.test_cached_moe_equals_composition_of_reference_routines(gpt_oss)
    json.dump(t._digest_cases(), open(os.path.join(HERE, "oracle_digests.json"), "w"), indent=1, sort_keys=True)
    print("wrote oracle_digests.json")


if __name__ == "__main__":
    main()
