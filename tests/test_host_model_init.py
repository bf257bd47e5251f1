"""CPU: the host-side model set-up (tscale_amd/host/model_init.cpp): InitAlibi against the reference's own InitModelDescr
(built into oracle/_ref) and against the oracle's restatement; ConvertMatrix (gpt/train/cpu_infer.cpp:94-121) against numpy and
by what it must satisfy; InitMatrixNormal (gpt/model_params/model_params.cpp:7-45) by its distribution and structure."""
import ctypes
import os

import numpy as np
import pytest

from oracle import pyoracle as orc
from tscale_amd import model_init as mi
from tscale_amd.attention import alibi_layer_schedule

REF_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libtsref.so")


@pytest.mark.parametrize("depth,wide", [(1, 64), (2, 128), (3, 4096), (12, 1024), (24, 2304), (25, 100), (48, 1024), (64, 512)])
def test_schedule(depth, wide):
    got = mi.init_alibi(depth, wide)
    ow, os_ = orc.init_alibi(depth, wide)
    assert got == list(zip([int(x) for x in ow], [float(x) for x in os_]))
    py = alibi_layer_schedule(depth, wide)
    assert [w for w, _ in got] == [w for w, _ in py] and np.allclose([s for _, s in got], [s for _, s in py], rtol=1e-7)
    if os.path.exists(REF_PATH):
        ref = ctypes.CDLL(REF_PATH)
        ref.ref_layer_schedule.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        w = (ctypes.c_longlong * 128)()
        s = (ctypes.c_float * 128)()
        n = ref.ref_layer_schedule(f"e512h4d{depth}w{wide}".encode(), 128, w, s)
        assert got == [(int(w[i]), float(s[i])) for i in range(n)]


def test_schedule_other_encodings():
    assert mi.init_alibi(6, 777, mi.ALIBI_NONE) == [(0, 0.0)] * 6
    assert mi.init_alibi(6, 777, mi.ALIBI_ABS_POS_ENCODING) == [(777, 0.0)] * 6


def test_convert_matrix():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((37, 64)) * 0.7).astype(np.float32)
    x[5, 7] = 30.0                                    # far outside: clamps to 127
    q, scale = mi.convert_matrix(x)
    sum2 = np.float32(0)
    for v in x.reshape(-1):                           # the reference's running float sum
        sum2 = np.float32(sum2 + np.float32(v * v))
    sko = np.sqrt(np.float32(sum2 / np.float32(x.size)))
    want_scale = np.float32(sko * np.float32(1.0 / 32))
    assert scale == want_scale
    mult = np.float32(1) / want_scale
    want = np.clip(np.rint(x * mult), -127, 127).astype(np.int8)
    assert np.array_equal(q, want) and q[5, 7] == 127 and q.min() >= -127
    # int8 * scale is the matrix again to half a step (where not clamped), and the int8 matrix has rms 32
    ok = np.abs(x) < 126 * scale
    assert np.abs(q * scale - x)[ok].max() <= 0.5 * scale * (1 + 1e-5)
    q2, _ = mi.convert_matrix(x[:5])                  # (no outlier in these rows)
    assert abs(np.sqrt((q2.astype(np.float64) ** 2).mean()) - 32) < 1.0
    # ties go to the even neighbour
    t = np.array([[0.5, 1.5, 2.5, -0.5, -1.5, 31.5, 32.0, 0.0]], dtype=np.float32)
    qt, st = mi.convert_matrix(t * np.float32(1))
    assert np.array_equal(qt, np.rint(t / st).clip(-127, 127).astype(np.int8))
    z, sz = mi.convert_matrix(np.zeros((4, 8), np.float32))
    assert sz == 0.0 and not z.any()


def test_init_matrix_normal():
    a = mi.init_matrix_normal(5, 1.0, 300, 512)
    b = mi.init_matrix_normal(5, 1.0, 300, 512)
    c = mi.init_matrix_normal(6, 1.0, 300, 512)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    assert abs(a.mean()) < 5e-3 and abs(a.std() - 0.5) < 5e-3          # normal values times sko * 0.5
    k = ((a / 0.5) ** 4).mean() / ((a / 0.5) ** 2).mean() ** 2
    assert abs(k - 3.0) < 0.1                                           # a normal distribution's kurtosis
    assert len(np.unique(np.abs(a))) <= 32768                          # a table of 65536 values in +- pairs
    assert np.array_equal(mi.init_matrix_normal(5, 2.0, 300, 512), a * 2)
    q, s = mi.random_int8_matrices(9, 3, 64, 128)
    assert q.shape == (3, 64, 128) and not np.array_equal(q[0], q[1]) and np.all(np.abs(s - 0.5 / 32) < 2e-3)
    qz, sz = mi.random_int8_matrices(9, 2, 8, 16, sko=0.0)              # COMBINER_INIT_ZERO
    assert not qz.any() and not sz.any()


@pytest.mark.parametrize("dim,heads,head_dim,relu_mult", [(2048, 16, 128, 1), (768, 12, 64, 1), (512, 4, 128, 2), (256, 2, 64, 3)])
def test_init_model_matrix_sizes(dim, heads, head_dim, relu_mult):
    """The matrices NTsAttn::InitModel makes have the sizes the layer (TLayerComputer, and the reference's AddLookupProduct)
    reads: the feed-forward block is HeadCount * 128 * ReluMult wide whatever the head width (model_dim.h:66)."""
    s = mi.init_model_shapes(dim, heads, head_dim, relu_mult)
    q_sum, relu = heads * head_dim, heads * 128 * relu_mult
    assert s["QK"] == s["QV"] == s["K"] == s["V"] == (q_sum, dim)
    assert s["Combiner"] == (dim, q_sum * 4)
    assert s["Expand"] == (relu, dim) and s["Contract"] == (dim, relu)


def test_init_alibi_respects_the_capacity():
    lib = mi.load()
    assert lib.tshost_init_alibi(mi.ALIBI_V3, 5, 100, None, None, 0) == 6      # an odd depth gains a layer
    w = np.full(8, -7, dtype=np.int32)
    s = np.full(8, -7.0, dtype=np.float32)
    assert lib.tshost_init_alibi(mi.ALIBI_V3, 5, 100, w.ctypes.data, s.ctypes.data, 4) == 6
    assert (w[4:] == -7).all() and (s[4:] == -7.0).all() and (w[:4] != -7).all()
