"""Validates the oracle's restatements against oracle/_ref/libtsref.so, which is compiled from the
reference's OWN sources (mask generation, layer schedule, e4m3 decode, constants).  Skipped where
that library has not been built (it needs the reference checkout at build time)."""
import ctypes
import os

import numpy as np
import pytest

from oracle import pyoracle as orc

REF_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libtsref.so")
pytestmark = pytest.mark.skipif(not os.path.exists(REF_PATH), reason="oracle/_ref not built")


@pytest.fixture(scope="module")
def ref():
    L = ctypes.CDLL(REF_PATH)
    L.ref_e4m3_to_float.restype = ctypes.c_float
    L.ref_att_dot_scale.restype = ctypes.c_float
    L.ref_attention_decay.restype = ctypes.c_float
    L.ref_attention_decay.argtypes = [ctypes.c_int, ctypes.c_float]
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.ref_layer_schedule.argtypes = [ctypes.c_char_p, ci, vp, vp]
    L.ref_spans.argtypes = [ctypes.c_char_p, ci, vp, vp, ci, ci, vp, vp, vp]
    L.ref_group_attention.argtypes = [ci, vp, vp, ci, vp, vp, vp]
    return L


def test_e4m3_decode_matches_reference(ref):
    tab = orc.e4m3_table()
    for c in range(256):
        want = ref.ref_e4m3_to_float(c if c < 128 else c - 256)
        if c == 0x80:
            # the reference's host decoder returns -2^-7 for the code of negative zero (its e == 0 branch
            # tests m > 0 only, util/fp8.h:17-20); the hardware and the oracle read it as -0
            assert want == -(2.0 ** -7) and tab[c] == 0
        elif (c & 0x7F) == 0x7F:
            # OCP NaN; the reference's formula gives +-480, the oracle follows the formula as well
            assert tab[c] == want
        else:
            assert tab[c] == want, c


def test_constants_match_reference(ref):
    for d in (64, 128, 192):
        assert orc.att_dot_scale(d) == ref.ref_att_dot_scale(d)
    assert ref.ref_attention_decay(7, 0.5) == -3.5


@pytest.mark.parametrize("depth,wide", [(12, 1024), (24, 2048), (1, 512), (6, 256), (42, 4096)])
def test_layer_schedule_matches_reference(ref, depth, wide):
    w = (ctypes.c_longlong * 128)()
    s = (ctypes.c_float * 128)()
    n = ref.ref_layer_schedule(f"e512h4d{depth}w{wide}".encode(), 128, w, s)
    ow, os_ = orc.init_alibi(depth, wide)
    assert n == len(ow)
    assert list(w)[:n] == list(ow) and list(s)[:n] == list(os_)


@pytest.mark.parametrize("doc_token", [-1, 3])
def test_spans_match_reference(ref, doc_token):
    rng = np.random.default_rng(0)
    frag_len = [1, 70, 300, 2, 129]
    n = sum(frag_len)
    tokens = rng.integers(0, 12, n).astype(np.int32)
    wide = 128
    descr = f"e512h4d12w{wide}".encode()
    # width ids of the reference's ALIBI_V3 table: 0 -> self only, 1 -> 1, 2 -> 64, 3 -> wide
    for width_id, window in ((0, 0), (1, 1), (2, 64), (3, wide)):
        st = np.zeros(n, np.int32); fi = np.zeros(n, np.int32); cnt = np.zeros(n, np.int32)
        fl = np.array(frag_len, np.int32)
        got_n = ref.ref_spans(descr, len(frag_len), fl.ctypes.data, tokens.ctypes.data, doc_token, width_id,
                              st.ctypes.data, fi.ctypes.data, cnt.ctypes.data)
        assert got_n == n and cnt.max() <= 1
        flags = None
        if doc_token >= 0:
            flags = (tokens == doc_token).astype(np.uint8)
        ost, ofi = orc.make_spans(frag_len, window, flags)
        has = cnt > 0
        assert np.array_equal(has, ofi >= ost)
        assert np.array_equal(st[has], ost[has]) and np.array_equal(fi[has], ofi[has])


def test_reference_tile_skip_list_covers_exactly_what_the_spans_need(ref):
    """GroupAttention<64,128> (the reference GPU kernel's tile-skip list) against the spans: every
    in-span key lies in some group's [start, finish + 127] range of its 64-row block."""
    st, fi = orc.make_spans([700, 300], 64)
    n = len(st)
    gb = np.zeros(4096, np.int32); gs = np.zeros(4096, np.int32); gf = np.zeros(4096, np.int32)
    ng = ref.ref_group_attention(n, st.ctypes.data, fi.ctypes.data, 4096, gb.ctypes.data, gs.ctypes.data, gf.ctypes.data)
    assert 0 < ng <= 4096
    for row in range(n):
        if fi[row] < st[row]:
            continue
        blk = row // 64
        cover = [(gs[i], gf[i] + 127) for i in range(ng) if gb[i] == blk]
        assert any(a <= st[row] and fi[row] <= b for a, b in cover), row
