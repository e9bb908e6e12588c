"""Pins the CPU restatement of crates/slai/src/models/sampler.rs:33-131 with closed forms and a library scan."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
from oracle import text_oracle as to  # noqa: E402


def test_uniform_distribution_is_floor_of_coin_times_n():
    n = 64                                          # 1/64 and its partial sums are exact in binary
    prob = np.full(n, 1.0 / n, dtype=np.float32)
    for coin in (0.0, 0.0156, 0.015625, 0.3, 0.5, 0.99, 0.999999):
        assert to.sample_mult(prob, coin) == int(np.floor(np.float32(coin) * n))
    assert to.sample(np.zeros(n, dtype=np.float32), 1.0, 0.0, 0.3) == int(0.3 * n)
    assert to.sample(np.zeros(n, dtype=np.float32), 1.0, 1.0, 0.3) == int(0.3 * n)     # topp >= 1: plain sampling


def test_rounding_fallback_is_the_last_index():
    prob = np.array([0.25, 0.25, 0.25], dtype=np.float32)      # does not sum to 1
    assert to.sample_mult(prob, 0.9) == 2


def test_temperature_zero_is_first_maximum():
    x = np.array([0.5, 3.0, -1.0, 3.0], dtype=np.float32)
    assert to.sample(x, 0.0, 0.9, 0.99) == 1


def test_dominant_logit_always_wins():
    x = np.full(1000, -20.0, dtype=np.float32)
    x[321] = 30.0
    for coin in (0.0, 0.5, 0.999):
        assert to.sample(x, 0.7, 0.95, coin) == 321
    for coin in (0.001, 0.5, 0.999):                            # without top-p a draw of exactly 0 picks index 0
        assert to.sample(x, 0.7, 0.0, coin) == 321
    assert to.sample(x, 0.7, 0.0, 0.0) == 0


def test_topp_on_powers_of_two():
    # sorted probabilities 1/2, 1/4, 1/8, ... (exact), scattered over the indices; topp = 0.8 keeps the first three:
    # 0.5, 0.75, 0.875 > 0.8, so the draw is coin * 0.875 against (0.5, 0.75, 0.875)
    n = 12
    where = [7, 2, 9, 0, 5, 11, 1, 3, 4, 6, 8, 10]
    prob = np.zeros(n, dtype=np.float32)
    for rank, i in enumerate(where):
        prob[i] = 2.0 ** -(rank + 1)
    prob[where[-1]] *= 2                                        # make the total exactly 1
    assert to.sample_topp(prob, 0.8, 0.5) == 7                  # r = 0.4375 < 0.5
    assert to.sample_topp(prob, 0.8, 0.6) == 2                  # r = 0.525
    assert to.sample_topp(prob, 0.8, 0.9) == 9                  # r = 0.7875
    assert to.sample_topp(prob, 0.8, 0.999999) == 9
    # a tiny topp keeps only the largest
    assert to.sample_topp(prob, 0.01, 0.999) == 7


def test_topp_equal_probabilities_keep_index_order():
    prob = np.array([0.125, 0.25, 0.25, 0.125, 0.25], dtype=np.float32)
    # order: 1, 2, 4 (0.25 each), then 0, 3; topp 0.7: 0.25, 0.5, 0.75 > 0.7 -> three kept, mass 0.75
    assert [to.sample_topp(prob, 0.7, c) for c in (0.1, 0.4, 0.9)] == [1, 2, 4]


def test_topp_cutoff_removes_small_candidates():
    # n = 5, topp = 0.5: cutoff = 0.125; the entry below it can never be drawn even though the mass never reaches topp
    # before it (0.2 + 0.2 < 0.5 ... the list ends at 0.45 and every candidate stays)
    prob = np.array([0.2, 0.1, 0.25, 0.0, 0.0], dtype=np.float32)
    assert to.sample_topp(prob, 0.5, 0.999) == 0                # candidates sorted: 2 (0.25), 0 (0.2); 0.45 <= 0.5


@pytest.mark.parametrize("n", [10, 257, 4000])
def test_scan_versions_agree_with_the_loops(n):
    rng = np.random.default_rng(n)
    for case in range(6):
        logits = (rng.standard_normal(n) * rng.choice([0.5, 2.0, 6.0])).astype(np.float32)
        for temperature, topp in ((0.7, 0.95), (1.0, 0.0), (0.3, 0.5), (1.5, 0.999), (0.0, 0.9)):
            for coin in rng.random(4).astype(np.float32):
                assert to.sample(logits, temperature, topp, coin) == to.sample_fast(logits, temperature, topp, coin)


def test_sample_mult_against_searchsorted():
    rng = np.random.default_rng(0)
    p = rng.random(500).astype(np.float32)
    p /= p.sum()
    cdf = np.cumsum(p, dtype=np.float32)
    for coin in rng.random(50).astype(np.float32):
        want = min(int(np.searchsorted(cdf, coin, side="right")), 499)
        assert to.sample_mult(p, coin) == want


def test_softmax_is_a_distribution():
    x = np.random.default_rng(1).standard_normal(300).astype(np.float32) * 5
    p = to.softmax_f32(x)
    assert abs(float(p.sum()) - 1.0) < 1e-5 and p.argmax() == x.argmax() and (p >= 0).all()
