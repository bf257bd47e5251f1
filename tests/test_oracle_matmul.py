"""CPU: the oracle's restatement of MulForward / AddScaled (gpt/train/cpu_infer.cpp:294-316) pinned against numpy's
integer matrix product (a library routine, not the oracle's loop) and against the extremes of the int8 range."""
import numpy as np
import pytest

from oracle import pyoracle as orc


@pytest.mark.parametrize("m,n,k", [(1, 1, 64), (5, 7, 128), (33, 100, 192), (130, 257, 2048)])
def test_matmul_i8_equals_numpy_int64_product(m, n, k):
    rng = np.random.default_rng(m * 1000 + n)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    want = a.astype(np.int64) @ w.astype(np.int64).T
    got = orc.matmul_i8(a, w)
    assert got.dtype == np.int32 and np.array_equal(got, want)


def test_matmul_i8_extremes_and_transposition():
    k = 4096
    a = np.full((2, k), 127, dtype=np.int8)
    a[1] = -127
    w = np.full((3, k), 127, dtype=np.int8)
    w[2, ::2] = -127
    got = orc.matmul_i8(a, w)
    assert got[0, 0] == 127 * 127 * k and got[1, 0] == -127 * 127 * k and got[0, 2] == 0
    # a weight ROW per output (MulForward's kqv[k]), not a column: an asymmetric case tells the two apart
    a = np.zeros((1, 64), dtype=np.int8); a[0, 3] = 2
    w = np.zeros((2, 64), dtype=np.int8); w[1, 3] = 5; w[0, 1] = 7
    assert orc.matmul_i8(a, w).tolist() == [[0, 10]]


def test_scaled_forms():
    rng = np.random.default_rng(9)
    a = rng.integers(-127, 128, (9, 128)).astype(np.int8)
    w = rng.integers(-127, 128, (11, 128)).astype(np.int8)
    sums = (a.astype(np.int64) @ w.astype(np.int64).T)
    scale = np.float32(0.0123)
    f = orc.matmul_i8(a, w, mode=1, scale=scale)
    assert f.dtype == np.float32 and np.array_equal(f, sums.astype(np.float32) * scale)
    state = rng.standard_normal((9, 11)).astype(np.float32)
    got = orc.matmul_i8(a, w, mode=2, scale=scale, out=state)
    assert np.array_equal(got, state + sums.astype(np.float32) * scale)   # one rounding per statement, as in AddScaled
    assert np.array_equal(orc.matmul_i8(a, w, mode=1, scale=1.0), sums.astype(np.float32))
