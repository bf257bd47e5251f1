"""Pins the oracle's element formats, quantisers, masks and dot products with checks that do not
restate the oracle's own formulas: first-principles tables, torch's float8 type, exact rational
arithmetic and brute force."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import pyoracle as orc


def ocp_e4m3_value(code):
    """OCP 8-bit float E4M3 (fn variant) from its definition: 1-4-3, bias 7, no inf."""
    s = -1 if code & 0x80 else 1
    e = (code >> 3) & 0xF
    m = code & 7
    if e == 0:
        return s * Fraction(m, 8) * Fraction(1, 2 ** 6)
    return s * (1 + Fraction(m, 8)) * Fraction(2) ** (e - 7)


def test_e4m3_decode_all_codes():
    tab = orc.e4m3_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    for c in range(256):
        if (c & 0x7F) == 0x7F:
            continue  # NaN in OCP; the reference decodes it as 480 and never produces it
        assert Fraction(float(tab[c])) == ocp_e4m3_value(c), c
        assert tab[c] == tt[c], c
    assert tab[0x7E] == 448.0 and tab[0x08] == 2.0 ** -6 and tab[0x01] == 2.0 ** -9


def test_e4m3_encode_roundtrip_ties_saturation():
    tab = orc.e4m3_table()
    codes = [c for c in range(256) if (c & 0x7F) != 0x7F]
    enc = orc.float_to_e4m3(tab[codes])
    for c, e in zip(codes, enc):
        if c == 0x80:
            assert e in (0x00, 0x80)
        else:
            assert e == c
    # ties between neighbouring positive codes go to the even code
    for c in range(0, 0x7E):
        mid = (float(tab[c]) + float(tab[c + 1])) / 2
        e = int(orc.float_to_e4m3([mid])[0])
        assert e == (c if c % 2 == 0 else c + 1), (c, mid, e)
        below = np.nextafter(np.float32(mid), np.float32(0))
        above = np.nextafter(np.float32(mid), np.float32(1e9))
        assert int(orc.float_to_e4m3([below])[0]) == c
        assert int(orc.float_to_e4m3([above])[0]) == c + 1
    assert list(orc.float_to_e4m3([448.0, 449.0, 463.9, 464.0, 1e9, np.inf])) == [0x7E] * 6
    assert list(orc.float_to_e4m3([-448.0, -1e9, -np.inf])) == [0xFE] * 3
    assert int(orc.float_to_e4m3([2.0 ** -10])[0]) == 0          # half of the smallest subnormal: tie to even (0)
    assert int(orc.float_to_e4m3([2.0 ** -10 * 1.01])[0]) == 1


def test_e4m3_encode_matches_torch_on_dense_sweep():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 100,
        rng.standard_normal(20000).astype(np.float32),
        rng.standard_normal(20000).astype(np.float32) * 0.01,
        np.linspace(-448, 448, 30001, dtype=np.float32),
    ])
    x = x[np.abs(x) <= 448]  # torch's cast does not saturate above the largest finite value
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = orc.float_to_e4m3(x)
    zero = (want & 0x7F) == 0
    assert np.array_equal(got[~zero], want[~zero])
    assert np.all((got[zero] & 0x7F) == 0)


def test_int8_rounding():
    x = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.4, 127.5, 300, -127.5, -128, -300, 0.49999, 3.7]
    want = [0, 2, 2, 0, -2, -2, 126, 127, 127, 127, -127, -127, -127, 0, 4]
    assert list(orc.float_to_i8(x)) == want


def test_bf16_roundtrip():
    x = np.random.default_rng(2).standard_normal(4096).astype(np.float32)
    bits = orc.float_to_bf16_bits(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bits, want)
    assert np.array_equal(orc.bf16_bits_to_float(bits), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    L = orc.lib()
    for i in range(64):
        assert L.tso_float_to_bf16(float(x[i])) == int(bits[i])
        assert L.tso_bf16_to_float(int(bits[i])) == orc.bf16_bits_to_float(bits[i:i + 1])[0]


@pytest.mark.parametrize("dtype", [orc.I8, orc.E4M3])
def test_quantize_rows_absmax(dtype):
    rng = np.random.default_rng(3)
    H, d, n = 3, 64, 50
    x = rng.standard_normal((n, H * d)).astype(np.float32)
    x[7, 64:128] = 0  # an all-zero (row, head)
    q, s = orc.quantize_rows(dtype, x, H)
    top = 127.0 if dtype == orc.I8 else 256.0
    tab = orc.e4m3_table()
    for t in range(n):
        for h in range(H):
            row = x[t, h * d:(h + 1) * d]
            amax = np.abs(row).max()
            if amax == 0:
                assert s[h, t] == 0 and not q[t, h * d:(h + 1) * d].any()
                continue
            assert s[h, t] == np.float32(amax) / np.float32(top)
            deq = q[t, h * d:(h + 1) * d].view(np.int8).astype(np.float32) if dtype == orc.I8 else tab[q[t, h * d:(h + 1) * d]]
            i = int(np.abs(row).argmax())
            assert abs(deq[i]) == top or (dtype == orc.I8 and abs(deq[i]) == 127)
            # reconstruction error bounded by half a step of the format
            step = 0.5 if dtype == orc.I8 else 2.0 ** (np.floor(np.log2(np.maximum(np.abs(deq), 2.0 ** -6))) - 3) / 2
            assert np.all(np.abs(deq - row / s[h, t]) <= step * 1.0001 + 1e-4)


def test_quantize_rows_bf16_matches_float_path():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((5, 2 * 128)).astype(np.float32)
    bits = orc.float_to_bf16_bits(x)
    q1, s1 = orc.quantize_rows(orc.I8, orc.bf16_bits_to_float(bits), 2)
    q2, s2 = orc.quantize_rows(orc.I8, bits, 2)
    assert np.array_equal(q1, q2) and np.array_equal(s1, s2)


def brute_force_pairs(seq_lens, window, flags):
    """Allowed (from,to) pairs from the rule in words: a token sees the `window` tokens before it,
    never itself, never across a sequence or document start; window 0 = itself only."""
    pairs = set()
    base = 0
    for n in seq_lens:
        for t in range(n):
            if window == 0:
                pairs.add((base + t, base + t))
                continue
            for to in range(t - 1, -1, -1):
                if t - to > window:
                    break
                pairs.add((base + t, base + to))
                if flags is not None and to > 0 and flags[base + to]:
                    break  # `to` starts a document: nothing earlier is visible
            # a document start at t itself hides everything before t
            if flags is not None and t > 0 and flags[base + t]:
                pairs -= {(base + t, base + to) for to in range(t)}
        base += n
    return pairs


@pytest.mark.parametrize("window", [0, 1, 3, 64, 1000])
def test_spans_match_brute_force(window):
    rng = np.random.default_rng(5)
    seq_lens = [1, 7, 70, 2, 33]
    n = sum(seq_lens)
    for flags in (None, (rng.random(n) < 0.08).astype(np.uint8)):
        st, fi = orc.make_spans(seq_lens, window, flags)
        got = {(f, t) for f in range(n) for t in range(st[f], fi[f] + 1)}
        assert got == brute_force_pairs(seq_lens, window, flags)


def test_init_alibi_schedule():
    # doc/model.md: first ~15% of layers width 1, then (0.5, 64) / (0, wide) interleaved
    w, s = orc.init_alibi(12, 1024)
    assert list(w) == [1, 1] + [64, 1024] * 5
    assert list(s) == [0, 0] + [0.5, 0] * 5
    w, s = orc.init_alibi(24, 2048)
    assert list(w) == [1] * 4 + [64, 2048] * 10 and list(s) == [0] * 4 + [0.5, 0] * 10
    w, s = orc.init_alibi(1, 777)
    assert list(w) == [777] and list(s) == [np.float32(0.1)]
    w, s = orc.init_alibi(5, 512)  # odd depth rounds up to whole pairs
    assert len(w) == 6


def test_dot_i8_exact_and_simd():
    rng = np.random.default_rng(6)
    for n in (64, 128, 192):
        for _ in range(50):
            a = rng.integers(-127, 128, n).astype(np.int8)
            b = rng.integers(-127, 128, n).astype(np.int8)
            want = int(np.dot(a.astype(np.int64), b.astype(np.int64)))
            assert orc.dot_i8(a, b) == want
            assert orc.dot_i8(a, b, simd=True) == want
        a = np.full(n, 127, np.int8)
        assert orc.dot_i8(a, a, simd=True) == 127 * 127 * n
        assert orc.dot_i8(a, -a, simd=True) == -127 * 127 * n


def test_dot_e4m3_is_exact_sum_rounded_once():
    rng = np.random.default_rng(7)
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    for n in (64, 128):
        for _ in range(30):
            a = rng.choice(codes, n)
            b = rng.choice(codes, n)
            exact = sum(ocp_e4m3_value(int(x)) * ocp_e4m3_value(int(y)) for x, y in zip(a, b))
            got = Fraction(float(orc.dot_e4m3(a, b)))
            f = np.float32(float(exact))  # Python rounds a Fraction to double correctly; double->float32 is then
            # exact unless the double rounding matters, which needs > 53 bits: sums here fit in 44 bits
            assert got == Fraction(float(f))


def test_softmax_buf_polynomial_is_close_to_exp2():
    rng = np.random.default_rng(8)
    for n in (1, 5, 8, 9, 64, 1000):
        x = (rng.standard_normal(n) * 4).astype(np.float32)
        logits = np.concatenate([[0.0], x]).astype(np.float32)
        w0, s0 = orc.softmax_buf(logits, 0)
        w1, s1 = orc.softmax_buf(logits, 1)
        m = max(0.0, float(x.max()))
        e = np.exp2(logits.astype(np.float64) - m)
        want = e / e.sum()
        assert np.allclose(w0, want, rtol=2e-6, atol=0)
        assert np.allclose(w1, want, rtol=1e-5, atol=1e-37)
        assert abs(float(w0.sum()) - 1) < 1e-5 and abs(float(w1.sum()) - 1) < 1e-5
    # huge negative logits are clamped, not NaN
    w1, _ = orc.softmax_buf(np.array([0, -1e30, -500], dtype=np.float32), 1)
    assert np.isfinite(w1).all() and abs(w1[0] - 1) < 1e-6
