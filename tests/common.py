"""Shared helpers for the parity tests: seeded inputs in the benchmark's shape and the error metric
the tolerance is stated in."""
import numpy as np

from oracle import pyoracle as orc

MAX_ABS_TOL = 2e-2   # on outputs rescaled to unit variance
MEAN_ABS_TOL = 2e-3


def seeded_normal(seed, shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def make_qkv(seed, n_tokens, n_heads, d, dtype):
    """N(0,1) Q,K,V [n_tokens, H*d], quantised per (token, head) row with the absmax rule."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(3):
        x = rng.standard_normal((n_tokens, n_heads * d)).astype(np.float32)
        out.append(orc.quantize_rows(dtype, x, n_heads))
    (q, qs), (k, ks), (v, vs) = out
    return q, qs, k, ks, v, vs


def unit_variance_errors(got, want):
    """max-abs and mean-abs error after dividing both by the std of the expected output."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    s = want.std()
    if s == 0:
        s = 1.0
    e = np.abs(got - want) / s
    return float(e.max()), float(e.mean())


def assert_within_tolerance(got, want, what=""):
    mx, mean = unit_variance_errors(got, want)
    assert mx <= MAX_ABS_TOL and mean <= MEAN_ABS_TOL, f"{what}: max {mx:.3e} mean {mean:.3e}"
    return mx, mean
