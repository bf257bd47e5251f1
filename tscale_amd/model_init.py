"""ctypes access to the host-side model set-up (tscale_amd/host/model_init.cpp): the InitAlibi layer schedule, InitMatrixNormal
and ConvertMatrix of the reference (gpt/model_params/model_dim.cpp:55-97, model_params.cpp:7-45, gpt/train/cpu_infer.cpp:94-121).
Plumbing for the tests and the benchmark, like capi.py."""
import ctypes as _c
import os

import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtshost.so")
ALIBI_NONE, ALIBI_V3, ALIBI_ABS_POS_ENCODING = 0, 1, 2
MODEL_DISCR_SCALE = 1.0 / 32
_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is missing: build it with `make -C tscale_amd/host`")
        L = _c.CDLL(LIB_PATH)
        L.tshost_init_alibi.restype = _c.c_int
        L.tshost_init_alibi.argtypes = [_c.c_int, _c.c_int, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int]
        L.tshost_init_model_shapes.restype = None
        L.tshost_init_model_shapes.argtypes = [_c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p]
        L.tshost_convert_matrix.restype = _c.c_float
        L.tshost_convert_matrix.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p]
        L.tshost_init_matrix_normal.argtypes = [_c.c_uint64, _c.c_float, _c.c_int64, _c.c_int64, _c.c_void_p]
        L.tshost_random_int8_matrices.argtypes = [_c.c_uint64, _c.c_float, _c.c_int64, _c.c_int64, _c.c_int, _c.c_void_p, _c.c_void_p]
        _lib = L
    return _lib


def init_alibi(depth, wide_limit_window, alibi=ALIBI_V3):
    """[(attention width, ALiBi slope)] per layer."""
    n = load().tshost_init_alibi(alibi, depth, wide_limit_window, None, None, 0)   # the schedule's own count (an odd depth gains a layer)
    w = np.zeros(n, dtype=np.int32)
    s = np.zeros(n, dtype=np.float32)
    got = load().tshost_init_alibi(alibi, depth, wide_limit_window, w.ctypes.data, s.ctypes.data, n)
    assert got == n
    return [(int(w[i]), float(s[i])) for i in range(got)]


def init_model_shapes(dim, head_count, head_dim, relu_mult=1):
    """(rows, cols) of the matrices NTsAttn::InitModel gives a layer: QK, QV, K, V, Combiner, Expand, Contract."""
    out = np.zeros((7, 2), dtype=np.int64)
    load().tshost_init_model_shapes(dim, head_count, head_dim, relu_mult, out.ctypes.data)
    return dict(zip(("QK", "QV", "K", "V", "Combiner", "Expand", "Contract"), (tuple(int(x) for x in r) for r in out)))


def convert_matrix(data):
    """float32 [y, x] -> (int8 [y, x], scale)."""
    data = np.ascontiguousarray(data, dtype=np.float32)
    out = np.empty(data.shape, dtype=np.int8)
    scale = load().tshost_convert_matrix(data.ctypes.data, data.shape[1], data.shape[0], out.ctypes.data)
    return out, float(scale)


def init_matrix_normal(seed, sko, y_size, x_size):
    out = np.empty((y_size, x_size), dtype=np.float32)
    load().tshost_init_matrix_normal(seed, sko, x_size, y_size, out.ctypes.data)
    return out


def random_int8_matrices(seed, n_matrices, y_size, x_size, sko=1.0):
    """n_matrices random matrices of a model (InitMatrixNormal, then ConvertMatrix): int8 [n, y, x] and their scales."""
    out = np.empty((n_matrices, y_size, x_size), dtype=np.int8)
    scales = np.empty(n_matrices, dtype=np.float32)
    load().tshost_random_int8_matrices(seed, sko, x_size, y_size, n_matrices, out.ctypes.data, scales.ctypes.data)
    return out, scales
