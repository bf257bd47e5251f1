"""CPU: the oracle's RoPE and per-head RMS normalisation (the producer of the attention operands,
gpt/att/rope.cpp:4-46, gpt/train/cpu_infer.cpp:358-391,486-499) pinned against the reference's own rope.cpp built
into oracle/_ref, against closed forms and a numpy restatement; and the library's host-side table builder."""
import ctypes
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tscale_amd import capi

REF = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libtsref.so")
VEC = np.float32(1.0 / 24)


def ref_lib():
    if not os.path.exists(REF):
        pytest.skip("oracle/_ref not built (no reference checkout)")
    lib = ctypes.CDLL(REF)
    lib.ref_fill_rope.argtypes = [ctypes.c_int, ctypes.c_longlong, ctypes.c_void_p]
    lib.ref_apply_rope.argtypes = [ctypes.c_int, ctypes.c_longlong, ctypes.c_float, ctypes.c_longlong, ctypes.c_int,
                                   ctypes.c_void_p]
    return lib


@pytest.mark.parametrize("width", [64, 128])
def test_rope_table_is_the_references(width):
    lib = ref_lib()
    want = np.empty((3000, width), np.float32)
    lib.ref_fill_rope(width, 3000, want.ctypes.data_as(ctypes.c_void_p))
    assert np.array_equal(orc.fill_rope(width, 3000), want)


@pytest.mark.parametrize("width,heads", [(64, 3), (128, 2)])
def test_apply_rope_is_the_references(width, heads):
    lib = ref_lib()
    rope = orc.fill_rope(width, 700)
    rng = np.random.default_rng(width)
    for t in (0, 1, 17, 699):
        for direction in (1.0, -1.0):
            v = rng.standard_normal(width * heads).astype(np.float32)
            want = v.copy()
            lib.ref_apply_rope(width, 700, direction, t, v.size, want.ctypes.data_as(ctypes.c_void_p))
            assert np.array_equal(orc.apply_rope(rope[t], direction, v, width), want)


def test_rope_is_a_rotation():
    rope = orc.fill_rope(128, 100)
    assert np.array_equal(rope[0, :32], np.ones(32, np.float32)) and not rope[0, 32:64].any()  # angle 0
    # first frequency is 1: position t has angle t
    assert abs(rope[3, 0] - np.cos(3.0)) < 1e-6 and abs(rope[3, 32] - np.sin(3.0)) < 1e-6
    v = np.random.default_rng(0).standard_normal(256).astype(np.float32)
    r = orc.apply_rope(rope[37], 1.0, v, 128)
    pair = lambda a: a.reshape(-1, 2, 32)  # blocks of 64: (k, k+32) couples
    assert np.allclose((pair(r) ** 2).sum(1), (pair(v) ** 2).sum(1), rtol=1e-5)
    assert np.allclose(orc.apply_rope(rope[37], -1.0, r, 128), v, atol=1e-5)


def test_library_table_builder_matches():
    if not os.path.exists(capi.LIB_PATH):
        pytest.fail("library not built")
    lib = capi.load()
    for width in (64, 128):
        got = np.empty((2500, width), np.float32)
        lib.tsattn_fill_rope_table(width, 2500, got.ctypes.data_as(ctypes.c_void_p))
        assert np.array_equal(got, orc.fill_rope(width, 2500))


def numpy_normalize(x, n_heads, dtype):
    """cpu_infer.cpp:358-391 once more, in numpy float32 scalar arithmetic."""
    n, hd = x.shape
    d = hd // n_heads
    q = np.zeros((n, hd), np.float32)
    sc = np.zeros((n_heads, n), np.float32)
    for t in range(n):
        for h in range(n_heads):
            v = x[t, h * d:(h + 1) * d].astype(np.float32)
            s = np.float32(0)
            for e in v:
                s = np.float32(s + np.float32(e * e))
            if s == 0:
                continue
            discr = np.float32(np.sqrt(np.float32(s / np.float32(d))) * VEC)
            mult = np.float32(np.float32(1) / discr)
            q[t, h * d:(h + 1) * d] = (v * mult).astype(np.float32)
            sc[h, t] = discr
    return q, sc


def test_normalize_closed_forms():
    # a constant head has sko = |c|: every value becomes 1/VEC_SCALE = 24, the scale |c|/24
    x = np.full((1, 128), -3.5, np.float32)
    q, s = orc.rope_normalize_rows(orc.I8, x, 1)
    assert (q.view(np.int8) == -24).all() and s[0, 0] == np.float32(3.5) * VEC
    # zero head: zeros and scale 0; the other head of the row is unaffected
    x = np.zeros((1, 128), np.float32); x[0, 64:] = 2.0
    q, s = orc.rope_normalize_rows(orc.I8, x, 2)
    assert not q[0, :64].any() and s[0, 0] == 0 and (q[0, 64:].view(np.int8) == 24).all()
    # one spike: sko = a/sqrt(d), value/scale = 24*sqrt(d) -> clamps to 127
    x = np.zeros((1, 64), np.float32); x[0, 5] = 7.0
    q, s = orc.rope_normalize_rows(orc.I8, x, 1)
    assert q.view(np.int8)[0, 5] == 127 and np.count_nonzero(q) == 1
    assert abs(s[0, 0] - 7.0 / 8 / 24) < 1e-7


@pytest.mark.parametrize("dtype", [orc.I8, orc.E4M3])
def test_normalize_against_numpy_and_scaling(dtype):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((9, 256)) * rng.uniform(0.01, 30, (9, 1))).astype(np.float32)
    q, s = orc.rope_normalize_rows(dtype, x, 2, scale_mult=0.37)
    y, want_s = numpy_normalize(x, 2, dtype)
    assert np.array_equal(s, (want_s * np.float32(0.37)).astype(np.float32))
    if dtype == orc.I8:
        want_q = np.clip(np.rint(y), -127, 127).astype(np.int8)
        assert np.array_equal(q.view(np.int8), want_q)
        deq = q.view(np.int8).astype(np.float32)
    else:
        deq = orc.e4m3_table()[q]
        assert np.abs(deq - y).max() <= np.abs(y).max() * 2.0 ** -4 + 2.0 ** -9
    # the dequantised head has the input's RMS (quantisation noise aside)
    rms = np.sqrt((deq.reshape(9, 2, 128) ** 2).mean(-1))
    assert np.allclose(rms, 24.0, rtol=0.02)
    # multiplying the input by a power of two moves only the scale
    q2, s2 = orc.rope_normalize_rows(dtype, x * np.float32(8), 2, scale_mult=0.37)
    assert np.array_equal(q2, q) and np.array_equal(s2, s * np.float32(8))


def test_int32_source_and_rope_composition():
    rng = np.random.default_rng(6)
    xi = rng.integers(-20000, 20000, (5, 128)).astype(np.int32)
    q, s = orc.rope_normalize_rows(orc.I8, xi, 2)
    q2, s2 = orc.rope_normalize_rows(orc.I8, xi.astype(np.float32), 2)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    # rope then normalise == normalise of the separately rotated rows
    rope = orc.fill_rope(64, 50)
    x = rng.standard_normal((5, 128)).astype(np.float32)
    pos = np.array([0, 3, 49, 7, 7], np.int32)
    q, s = orc.rope_normalize_rows(orc.I8, x, 2, pos=pos, rope=rope)
    rot = np.stack([orc.apply_rope(rope[p], 1.0, x[i], 64) for i, p in enumerate(pos)])
    q2, s2 = orc.rope_normalize_rows(orc.I8, rot, 2)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)


def test_kv_product_against_numpy():
    """KVProduct (cpu_infer.cpp:320-337): index shuffle z ^ blk inside each head, product, int8 rounding."""
    rng = np.random.default_rng(12)
    n, H, d = 5, 3, 64
    k = rng.integers(-127, 128, (n, H * d)).astype(np.int8)
    val = (rng.standard_normal((n, H * d)) * 0.3).astype(np.float32)
    kv = orc.kv_product(k, val, H)
    assert kv.shape == (n, H * d * 4)
    k3 = k.reshape(n, H, d).astype(np.float32); v3 = val.reshape(n, H, d)
    z = np.arange(d)
    for blk in range(4):
        want = np.clip(np.rint(k3[:, :, z ^ blk] * v3), -127, 127).astype(np.int8)
        assert np.array_equal(kv.reshape(n, H, 4, d)[:, :, blk], want)
    # blk 0 is the plain product; with a constant value the blocks are permutations of block 0
    kv1 = orc.kv_product(k, np.full_like(val, 0.5), H).reshape(n, H, 4, d)
    for blk in range(4):
        assert np.array_equal(kv1[:, :, blk], kv1[:, :, 0][:, :, z ^ blk])
    # clamp
    big = orc.kv_product(np.full((1, 64), 100, np.int8), np.full((1, 64), 3.0, np.float32), 1)
    assert (big == 127).all()
