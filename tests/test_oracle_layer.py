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


# ---- the composition as a whole --------------------------------------------------------------------------------------
# The reference checks its int8 layer against its real-valued model (NCPUInfer::Check, gpt/train/cpu_infer.cpp:625-685):
# int8 values times their scales are approximations of real vectors, and every rounding step can be left out.  What
# follows is that real-valued layer in float64, written from gpt/train/cpu_infer.cpp:465-527 with NormalizeState
# (:358-391) as a division by rms * VEC_SCALE, ApplyRope (gpt/att/rope.cpp:28-46) as a complex rotation, the attention
# (:413-460) as an ordinary softmax with one zero key, KVProduct (:320-337) as a product of k shuffled by z ^ blk with the
# attention output, MulForward / AddScaled (:294-316) as matrix products.  Nothing is rounded to int8 anywhere, and the
# KV cache holds real vectors.  The oracle must agree with it to within the rounding of its int8 vectors -- and a layer
# with k and v exchanged, a scale computed from the wrong width, a dropped VEC_SCALE or the ReLU in front of the
# normalisation must not.
VS = 1.0 / 24
LOG2 = 0.693147


def _rms_norm(x, groups):
    g = x.reshape(groups, -1)
    rms = np.sqrt((g * g).mean(axis=1, keepdims=True))
    return (g / (rms * VS)).reshape(-1), (rms[:, 0] * VS)


def _rotate(x, rope_row, d):
    out = x.copy().reshape(-1, d)
    for blk in range(0, d, 64):
        z = out[:, blk:blk + 32] + 1j * out[:, blk + 32:blk + 64]
        z = z * (rope_row[blk:blk + 32] + 1j * rope_row[blk + 32:blk + 64])
        out[:, blk:blk + 32], out[:, blk + 32:blk + 64] = z.real, z.imag
    return out.reshape(-1)


def real_layer(mats, scales, width, slope, t, rope, state, cache, mutate=None):
    """One token of one sequence.  cache: list of (qv vector [H*D], v vector [H*D]) of the rows before it."""
    W = {n: m.astype(np.float64) for n, m in mats.items()}
    qv_scale, comb_scale, contr_scale = scales
    if mutate == "key_scale_10pct":
        qv_scale *= 1.1
    if mutate == "combiner_scale_10pct":
        comb_scale *= 1.1
    if mutate == "contract_scale_10pct":
        contr_scale *= 1.1
    dim = state.size
    n, _ = _rms_norm(state, dim // 128)
    qk, qv, k, v = W["qk"] @ n, W["qv"] @ n, W["k"] @ n, W["v"] @ n
    qk, qv = _rotate(qk, rope[t], D), _rotate(qv, rope[t], D)
    qk, _ = _rms_norm(qk, H)
    k, _ = _rms_norm(k, H)
    v, _ = _rms_norm(v, H)
    # the cache keeps qv itself (the int8 path: its normalised form and the scale that undoes the normalisation)
    key_mult = qv_scale * VS * np.sqrt(1.0 / (D if mutate == "dot_scale_of_head" else dim))
    if mutate == "drop_vec_scale":
        key_mult = qv_scale * np.sqrt(1.0 / dim)
    cache.append((qv * key_mult, v))
    cur = len(cache) - 1
    keys = [cur] if width == 0 else list(range(cur - 1, cur - 1 - min(cur, width), -1))
    att_scale = np.sqrt(1.0 / D) * (0.5 / LOG2)
    val = np.zeros(H * D)
    for h in range(H):
        sl = slice(h * D, (h + 1) * D)
        logits = np.array([0.0] + [qk[sl] @ cache[to][0][sl] * att_scale * VS - slope * (cur - to) for to in keys])
        w = np.exp2(logits - logits.max())
        w /= w.sum()
        for z, to in enumerate(keys):
            val[sl] += w[z + 1] * VS * cache[to][1][sl]
    a, b = (v, k) if mutate == "swap_k_v" else (k, v)
    del b
    kv = np.empty(H * D * 4)
    for h in range(H):
        for blk in range(4):
            z = np.arange(D)
            kv[(h * 4 + blk) * D:(h * 4 + blk + 1) * D] = a[h * D + (z ^ blk)] * val[h * D + z]
    state = state + (W["combiner"] @ kv) * (comb_scale * VS * np.sqrt(1.0 / kv.size))
    n2, _ = _rms_norm(state, dim // 128)
    relu_src = W["expand"] @ n2
    if mutate == "relu_before_norm":
        relu, _ = _rms_norm(np.maximum(relu_src, 0.0), H)
    else:
        relu = np.maximum(_rms_norm(relu_src, H)[0], 0.0)
    state = state + (W["contract"] @ relu) * (contr_scale * VS * np.sqrt(1.0 / relu.size))
    return state, val


def _run_both(mutate, n_tokens=6, width=100, slope=0.0, seed=21, rms=False, scales=(0.04, 0.03, 0.05)):
    """n_tokens tokens of B sequences through the oracle (one shared cache object, as the reference keeps it) and through
    the real-valued layer; both start every token from the oracle's state, so rounding does not pile up over tokens.
    Returns the largest differences of the new state's update and of the attention output, relative to their rms; with
    rms=True the rms of the update's difference over all tokens and sequences relative to the update's rms (the int8
    rounding averages out in it, a scale that is off does not)."""
    mats = make_layer(seed)
    rng = np.random.default_rng(seed + 1)
    state = rng.standard_normal((B, DIM)).astype(np.float32)
    k = np.zeros((B, H, MAXLEN, D), dtype=np.uint8)
    v = np.zeros((B, H, MAXLEN, D), dtype=np.uint8)
    ks = np.zeros((B, H, MAXLEN), dtype=np.float32)
    cl = np.zeros(B, dtype=np.int32)
    rope = orc.fill_rope(D, 64)
    caches = [[] for _ in range(B)]
    worst_state, worst_val = 0.0, 0.0
    sq_err, sq_ref = 0.0, 0.0
    for tok in range(n_tokens):
        t = np.full(B, tok, dtype=np.int32)
        new_state, val = orc.add_lookup_product(mats, scales, width, slope, H, D, t, rope, state, k, v, ks, cl)
        for b in range(B):
            want_state, want_val = real_layer(mats, scales, width, slope, tok, rope.astype(np.float64), state[b].astype(np.float64),
                                              caches[b], mutate)
            upd, want_upd = new_state[b] - state[b], want_state - state[b]
            worst_state = max(worst_state, np.abs(upd - want_upd).max() / np.sqrt((want_upd ** 2).mean()))
            sq_err += float(((upd - want_upd) ** 2).sum())
            sq_ref += float((want_upd ** 2).sum())
            if tok > 0:
                worst_val = max(worst_val, np.abs(val[b] - want_val).max() / (np.sqrt((want_val ** 2).mean()) + 1e-30))
        state = new_state
    if rms:
        return np.sqrt(sq_err / sq_ref)
    return worst_state, worst_val


def test_layer_agrees_with_its_real_valued_form():
    for width, slope in ((100, 0.0), (2, 0.5), (0, 0.0)):
        ws, wv = _run_both(None, width=width, slope=slope)
        assert ws < 0.15 and wv < 0.15, (width, slope, ws, wv)


@pytest.mark.parametrize("mutate", ["swap_k_v", "dot_scale_of_head", "drop_vec_scale", "relu_before_norm"])
def test_a_wrong_composition_does_not(mutate):
    good_s, good_v = _run_both(None)
    bad_s, bad_v = _run_both(mutate)
    assert max(bad_s / good_s, bad_v / good_v) > 4.0, (mutate, good_s, good_v, bad_s, bad_v)


@pytest.mark.parametrize("mutate", ["key_scale_10pct", "combiner_scale_10pct", "contract_scale_10pct"])
def test_a_scale_ten_percent_off_shows(mutate):
    """The largest-element figure of the state lets a mis-scaling of 10 % through.  For the two matrix scales that act on
    the state the rms over everything does not: the int8 rounding leaves about 2 % there and averages out, a scale that is
    off adds its share in full.  The key scale acts on the logits: the attention output's largest difference doubles."""
    if mutate == "key_scale_10pct":
        _, good = _run_both(None)
        _, bad = _run_both(mutate)
        assert good < 0.08 and bad > 1.6 * good, (mutate, good, bad)
        return
    good = _run_both(None, rms=True)
    bad = _run_both(mutate, rms=True)
    assert good < 0.05, good
    assert bad > 1.5 * good, (mutate, good, bad)
