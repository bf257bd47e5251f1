"""CPU: the oracle's AddLookupProduct (gpt/train/cpu_infer.cpp:465-527).  Its parts are pinned one by one elsewhere;
what can be said of the composition without retyping it: the input state's scale does not matter to the attention half
(the state is normalised first, :476), zero combiner and contract matrices leave the state alone while the cache still grows, the first token
of a sequence sees no keys, and the two updates are linear in their matrix scales."""
import numpy as np
import pytest

from oracle import pyoracle as orc

H, D, DIM, MAXLEN, B = 2, 64, 256, 8, 3


def make_layer(seed, zero=()):
    rng = np.random.default_rng(seed)
    qsum, relu = H * D, H * D
    shapes = {"qk": (qsum, DIM), "qv": (qsum, DIM), "k": (qsum, DIM), "v": (qsum, DIM), "combiner": (DIM, qsum * 4),
              "expand": (relu, DIM), "contract": (DIM, relu)}
    mats = {n: np.clip(np.rint(rng.standard_normal(s) * 32), -127, 127).astype(np.int8) for n, s in shapes.items()}
    for n in zero:
        mats[n][:] = 0
    return mats


def fresh_cache(seed, lens):
    rng = np.random.default_rng(seed)
    k = rng.integers(0, 256, (B, H, MAXLEN, D)).astype(np.uint8)
    v = rng.integers(0, 256, (B, H, MAXLEN, D)).astype(np.uint8)
    ks = ((rng.random((B, H, MAXLEN)) + 0.5) * 1e-3).astype(np.float32)
    return k, v, ks, np.array(lens, dtype=np.int32)


def run(mats, scales, state, lens, width=100, slope=0.0, seed=5):
    k, v, ks, cl = fresh_cache(seed, lens)
    rope = orc.fill_rope(D, 64)
    t = cl.copy()
    out, val = orc.add_lookup_product(mats, scales, width, slope, H, D, t, rope, state, k, v, ks, cl)
    return out, val, (k, v, ks, cl)


def test_input_scale_does_not_matter_to_the_attention_half():
    """The state is normalised before the projections (:476), so the attention output, the rows put into the cache and
    the combiner's update do not depend on the state's scale (the feed-forward half does: it normalises the sum of the
    state and that update)."""
    mats = make_layer(1, zero=("contract",))
    state = np.random.default_rng(2).standard_normal((B, DIM)).astype(np.float32)
    a, val_a, cache_a = run(mats, (0.03, 0.03, 0.03), state, [2, 5, 0])
    b, val_b, cache_b = run(mats, (0.03, 0.03, 0.03), state * 4, [2, 5, 0])
    assert np.array_equal(val_a, val_b)
    for x, y in zip(cache_a, cache_b):
        assert np.array_equal(x, y)
    # the update is the same; only its addition to a state four times as large rounds differently
    assert np.abs((b - 4 * state) - (a - state)).max() < 1e-5 * np.abs(a).max()
    assert np.abs(a - state).max() > 1e-3, "the layer changed nothing: the test would say nothing"


def test_zero_output_matrices_leave_the_state_but_fill_the_cache():
    mats = make_layer(3, zero=("combiner", "contract"))
    state = np.random.default_rng(4).standard_normal((B, DIM)).astype(np.float32)
    out, val, (k, v, ks, cl) = run(mats, (0.03, 0.03, 0.03), state, [2, 7, 8])
    assert np.array_equal(out, state)
    assert cl.tolist() == [3, 8, 8]            # the full cache drops the row
    k0, v0, ks0, _ = fresh_cache(5, [2, 7, 8])
    assert not np.array_equal(k[0, :, 2], k0[0, :, 2]) and not np.array_equal(v[1, :, 7], v0[1, :, 7])
    assert np.array_equal(k[2], k0[2]) and np.array_equal(ks[2], ks0[2])
    assert np.array_equal(k[0, :, 3:], k0[0, :, 3:])   # only row cache_len was written


def test_first_token_sees_no_keys_and_width_zero_sees_itself():
    mats = make_layer(6)
    state = np.random.default_rng(7).standard_normal((B, DIM)).astype(np.float32)
    _, val, _ = run(mats, (0.03, 0.03, 0.03), state, [0, 0, 3])
    assert not val[0].any() and not val[1].any() and val[2].any()
    _, val0, _ = run(mats, (0.03, 0.03, 0.03), state, [0, 0, 3], width=0)
    assert val0[0].any(), "width 0: the token attends to its own row (cpu_infer.cpp:430-433)"


def test_updates_are_linear_in_the_matrix_scales():
    state = np.random.default_rng(9).standard_normal((B, DIM)).astype(np.float32)
    only_combiner = make_layer(8, zero=("contract",))
    a, _, _ = run(only_combiner, (0.03, 0.02, 0.0), state, [3, 4, 5])
    b, _, _ = run(only_combiner, (0.03, 0.04, 0.0), state, [3, 4, 5])
    assert np.abs((b - state) - 2 * (a - state)).max() < 1e-5 * np.abs(a - state).max() + 1e-6
    only_ffn = make_layer(8, zero=("combiner",))
    a, _, _ = run(only_ffn, (0.03, 0.0, 0.02), state, [3, 4, 5])
    b, _, _ = run(only_ffn, (0.03, 0.0, 0.04), state, [3, 4, 5])
    assert np.abs((b - state) - 2 * (a - state)).max() < 1e-5 * np.abs(a - state).max() + 1e-6
    assert np.abs(a - state).max() > 1e-3
