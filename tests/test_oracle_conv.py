"""Pins of uk_oracle_conv_nchwc (CPU only): an independent numpy statement of
the convolution, the early-return cases of conv_nchwc.c:42-53, and buffer-for-
buffer equality with the compiled reference on the reference test's own case
grid (tools/conv_nchwc_test.c:187-226), generic path and AVX-512 16x16 tile."""
import numpy as np
import pytest

import conv_testing as C


def test_conv_oracle_equals_numpy_statement(oracle):
    n = 0
    for ci, c in enumerate(C.cases(seed=5)):
        rng = np.random.default_rng(ci)
        inp, flt, out0 = C.buffers(c, rng)
        got = out0.copy()
        C.run(oracle, c, inp, flt, got)
        early = (c.N == 0 or c.OC_outer == 0 or c.OH == 0 or c.OW == 0 or
                 ((c.IC_outer == 0 or c.FH == 0 or c.FW == 0) and c.flags & C.CONV_ACCUMULATE))
        if early:
            assert np.array_equal(got, out0), c.label()
            continue
        want = C.numpy_conv(c, inp, flt, out0)
        assert np.array_equal(C.dense_output(c, got).astype(np.float64), want), c.label()
        # nothing outside the output pixels is written
        mask = np.ones(out0.size, bool)
        for nn in range(c.N):
            for oc in range(c.OC_outer):
                for oh in range(c.OH):
                    b = c.offsets[2] + nn * c.out_strides[0] + oc * c.out_strides[1] + oh * c.out_strides[2]
                    mask[b:b + c.OW * c.k0] = False
        assert np.array_equal(got[mask], out0[mask]), c.label()
        n += 1
    assert n > 100


def test_conv_oracle_equals_compiled_reference(oracle, reference):
    for features in (False, True):
        reference.use_host_cpu_features(features)
        for ci, c in enumerate(C.cases(seed=9)):
            rng = np.random.default_rng(1000 + ci)
            for exact in (True, False):
                if not exact and features and (c.k0, c.c0) == (16, 16):
                    continue   # the AVX-512 tile uses FMA: same sums only on exact inputs
                inp, flt, out0 = C.buffers(c, rng, exact=exact)
                a, b = out0.copy(), out0.copy()
                C.run(oracle, c, inp, flt, a)
                C.run(reference, c, inp, flt, b)
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (c.label(), features, exact)
    reference.use_host_cpu_features(False)


def test_conv_oracle_matches_committed_reference_digests(oracle):
    """Digests written by tests/golden/make_golden.py from the compiled
    reference (generic path); checks the oracle where oracle/_ref is absent."""
    import json
    import os
    from golden import make_golden as G
    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_conv.json")) as f:
        want = json.load(f)
    got = G.conv_digests(oracle)
    assert got.keys() == want.keys() and len(got) == 320
    bad = [k for k in got if got[k] != want[k]]
    assert not bad, bad[:5]
