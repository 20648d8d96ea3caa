"""The host-side sampler of forward_token's non-greedy branch (crates/ksearch_gemma/src/sample.rs): the reference's
own unit tests restated for the oracle and for the library's function, the two against each other, and the draw
against the closed-form distribution.  No GPU work."""
import numpy as np

import oracle
from ksearch_amd import hip

BOTH = (oracle.sample_softcap_min_p, hip.sample_softcap_min_p)


def test_reference_unit_tests_restated():
    for f in BOTH:
        # sample.rs:94-98
        assert f(np.array([1.0, 9.0, 3.0], np.float32), 30.0, 0.0, 0.05, 1) == 1
        # :100-108: a peaked distribution keeps only the peak under min-p
        assert {f(np.array([0.0, 20.0, 0.0], np.float32), 30.0, 1.0, 0.05, s) for s in range(1, 64)} == {1}
        # :110-117: near-ties after the soft cap are both drawn, the far one never
        counts = np.bincount([f(np.array([8.0, 8.05, 0.0], np.float32), 30.0, 1.0, 0.05, s) for s in range(1, 256)], minlength=3)
        assert counts[0] > 0 and counts[1] > 0 and counts[2] == 0


def test_library_equals_oracle_and_rules():
    rng = np.random.default_rng(800)
    for trial in range(40):
        n = int(rng.integers(1, 3000))
        x = (rng.standard_normal(n) * rng.choice([0.5, 5.0, 60.0])).astype(np.float32)
        for temp, min_p in ((0.0, 0.05), (0.7, 0.05), (1.0, 0.0), (2.0, 0.3)):
            for seed in (0, 1, 12345, 2 ** 32 - 1):
                assert hip.sample_softcap_min_p(x, 30.0, temp, min_p, seed) == oracle.sample_softcap_min_p(x, 30.0, temp, min_p, seed)
        # greedy = the device argmax's rule; cap 0 switches the soft cap off
        assert hip.sample_softcap_min_p(x, 30.0, 0.0) == oracle.softcap_argmax(x, 30.0)
        assert hip.sample_softcap_min_p(x, 0.0, 0.0) == int(np.argmax(x))
    # seeds differing in bit 0 only draw the same id (the generator's state is seed | 1)
    x = rng.standard_normal(500).astype(np.float32)
    assert all(hip.sample_softcap_min_p(x, 30.0, 1.0, 0.0, 2 * k) == hip.sample_softcap_min_p(x, 30.0, 1.0, 0.0, 2 * k + 1) for k in range(50))


def test_draw_follows_the_filtered_softmax():
    x = np.array([2.0, 1.0, 0.0, -1.0, -6.0], np.float32)
    cap, temp, min_p = 30.0, 0.8, 0.05
    y = cap * np.tanh(x.astype(np.float64) / cap)
    p = np.exp((y - y.max()) / temp)
    p /= p.sum()
    p[p < min_p * p.max()] = 0.0          # the last id falls under the min-p bar
    p /= p.sum()
    draws = np.bincount([hip.sample_softcap_min_p(x, cap, temp, min_p, s) for s in range(1, 8001, 2)], minlength=5) / 4000.0
    assert draws[4] == 0.0 and np.abs(draws - p).max() < 0.03
