"""CPU: the oracle's embedding sum and final softmax (gpt/train/cpu_infer.cpp:552-582, :340-355) against library
routines and properties."""
import numpy as np
from scipy.special import softmax

from oracle import pyoracle as orc


def test_embed_rows_is_a_gather_and_sum():
    rng = np.random.default_rng(1)
    embed = rng.integers(-127, 128, (50, 64)).astype(np.int8)
    labels = np.array([[3, 7, -1], [49, 49, 0], [-1, -1, -1], [12, 50, 1]], dtype=np.int32)   # -1 and 50: empty slots
    got = orc.embed_rows(labels, embed, 0.125)       # a power of two: every product and sum is exact
    want = np.zeros((4, 64))
    for r, row in enumerate(labels):
        for l in row:
            if 0 <= l < 50:
                want[r] += embed[l] * 0.125
    assert np.array_equal(got, want.astype(np.float32))
    assert not got[2].any()


def test_softmax_rows_is_a_base_2_softmax_with_a_floor_on_the_maximum():
    rng = np.random.default_rng(2)
    vec = (rng.standard_normal((5, 1000)) * 4000).astype(np.int32)
    bias = rng.standard_normal(1000).astype(np.float32)
    scale = 1e-3
    prob, arg = orc.softmax_rows(vec, scale, bias)
    w = vec.astype(np.float64) * np.float32(scale) + bias
    want = softmax(w * np.log(2.0), axis=1)          # 2^w / sum 2^w
    assert np.abs(prob - want).max() < 1e-6 and np.abs(prob / want - 1).max() < 1e-4
    assert np.abs(prob.sum(axis=1) - 1).max() < 1e-5
    assert np.array_equal(arg, w.argmax(axis=1))
    # the reference's polynomial exp2 stays within 1e-5 of it
    prob_poly, _ = orc.softmax_rows(vec, scale, bias, exp2_mode=1)
    assert np.abs(prob_poly / want - 1).max() < 1e-4
    # shifting every logit (through the bias) changes nothing while the largest stays above 0 ...
    prob2, arg2 = orc.softmax_rows(vec, scale, bias + 3.0)
    assert np.abs(prob2 - prob).max() < 1e-6 and np.array_equal(arg2, arg)
    # ... and all-negative logits are taken relative to 0, not to their maximum: still a distribution
    prob3, _ = orc.softmax_rows(-np.abs(vec) - 50000, scale, None)
    assert np.abs(prob3.sum(axis=1) - 1).max() < 1e-5
    # ties: the first index wins
    tie = np.zeros((1, 16), dtype=np.int32); tie[0, [5, 9]] = 7
    assert orc.softmax_rows(tie, 1.0)[1].tolist() == [5]


def test_sample_rows_draws_from_the_tempered_distribution():
    """SampleFromDistr (cpu_infer.cpp:585-599) is the Gumbel-max trick: argmax of log p / T + Gumbel noise is a draw
    from p^(1/T) normalised.  A wrong sign, a missing logarithm or a dropped temperature changes the frequencies."""
    p = np.array([0.4, 0.25, 0.15, 0.1, 0.07, 0.03], dtype=np.float32)
    draws = 200000
    prob = np.tile(p, (draws, 1))
    for temperature in (1.0, 2.0):
        choice = orc.sample_rows(prob, temperature, seed=17, offset=int(temperature * 1000))
        want = p.astype(np.float64) ** (1.0 / temperature)
        want /= want.sum()
        freq = np.bincount(choice, minlength=6) / draws
        sigma = np.sqrt(want * (1 - want) / draws)
        assert (np.abs(freq - want) < 4.5 * sigma).all(), (temperature, freq, want)
    # a tiny temperature: the noise no longer matters, the largest probability wins; ties go to the first index
    rng = np.random.default_rng(5)
    q = rng.random((64, 300)).astype(np.float32)
    q[np.arange(64), rng.integers(0, 300, 64)] = 3.0           # a clear winner per row
    q /= q.sum(axis=1, keepdims=True)
    assert np.array_equal(orc.sample_rows(q, 1e-3, seed=3), q.argmax(axis=1))
    # words handed in by the caller and the counter generator's own words are the same thing
    words = np.array([[orc.mix32(99, 7 + r * 300 + k) for k in range(300)] for r in range(4)], dtype=np.uint32)
    assert np.array_equal(orc.sample_rows(q[:4], 0.8, rnd=words), orc.sample_rows(q[:4], 0.8, seed=99, offset=7))
    # probability zero is never chosen
    z = np.zeros((3, 50), dtype=np.float32); z[:, 31] = 1.0
    assert (orc.sample_rows(z, 1.0, seed=1) == 31).all()
