"""numpy front end of libtsattn_oracle.so (the CPU checker).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py.  The product package (tscale_amd) never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtsattn_oracle.so")

I8 = 0
E4M3 = 1

_c = ctypes
_i64 = _c.c_int64
_f32 = _c.c_float
_int = _c.c_int
_vp = _c.c_void_p


def build():
    """Compile the checker with gcc (make in this directory)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "libtsattn_oracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.tso_e4m3_to_float.restype = _f32
        L.tso_e4m3_to_float.argtypes = [_c.c_uint8]
        L.tso_float_to_e4m3.restype = _c.c_uint8
        L.tso_float_to_e4m3.argtypes = [_f32]
        L.tso_float_to_i8.restype = _c.c_int8
        L.tso_float_to_i8.argtypes = [_f32]
        L.tso_bf16_to_float.restype = _f32
        L.tso_bf16_to_float.argtypes = [_c.c_uint16]
        L.tso_float_to_bf16.restype = _c.c_uint16
        L.tso_float_to_bf16.argtypes = [_f32]
        L.tso_att_dot_scale.restype = _f32
        L.tso_att_dot_scale.argtypes = [_int]
        L.tso_quantize_rows.restype = None
        L.tso_quantize_rows.argtypes = [_int, _vp, _i64, _i64, _int, _int, _vp, _i64, _vp, _i64]
        L.tso_quantize_rows_bf16.restype = None
        L.tso_quantize_rows_bf16.argtypes = [_int, _vp, _i64, _i64, _int, _int, _vp, _i64, _vp, _i64]
        L.tso_make_spans.restype = None
        L.tso_make_spans.argtypes = [_i64, _vp, _vp, _i64, _vp, _vp]
        L.tso_init_alibi.restype = _int
        L.tso_init_alibi.argtypes = [_int, _i64, _int, _vp, _vp]
        L.tso_dot_i8.restype = _c.c_int32
        L.tso_dot_i8.argtypes = [_vp, _vp, _int]
        L.tso_dot_i8_simd.restype = _c.c_int32
        L.tso_dot_i8_simd.argtypes = [_vp, _vp, _int]
        L.tso_dot_e4m3.restype = _f32
        L.tso_dot_e4m3.argtypes = [_vp, _vp, _int]
        L.tso_qk_accum.restype = None
        L.tso_qk_accum.argtypes = [_int, _vp, _i64, _vp, _i64, _int, _int, _i64, _i64, _i64, _i64, _vp]
        L.tso_prefill_f32.restype = None
        L.tso_prefill_f32.argtypes = [_i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp]
        L.tso_prefill_q8.restype = None
        L.tso_prefill_q8.argtypes = [_int, _i64, _int, _int, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64,
                                     _f32, _f32, _f32, _vp, _vp, _f32, _vp, _i64, _vp, _int]
        L.tso_decode.restype = None
        L.tso_decode.argtypes = [_int, _i64, _int, _int, _vp, _vp, _f32, _vp, _vp, _i64, _i64, _i64,
                                 _vp, _vp, _i64, _i64, _f32, _f32, _vp, _i64, _f32, _int, _int, _vp,
                                 _vp, _i64, _int]
        L.tso_softmax_buf.restype = _f32
        L.tso_softmax_buf.argtypes = [_vp, _int, _int, _vp]
        L.tso_simd_level.restype = _int
        L.tso_max_threads.restype = _int
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _c_arr(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


# ---- formats ---------------------------------------------------------------------------------
def e4m3_table():
    L = lib()
    return np.array([L.tso_e4m3_to_float(i) for i in range(256)], dtype=np.float32)


def float_to_e4m3(x):
    L = lib()
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    xf, of = x.ravel(), out.ravel()
    for i in range(xf.size):
        of[i] = L.tso_float_to_e4m3(float(xf[i]))
    return out


def float_to_i8(x):
    L = lib()
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.int8)
    xf, of = x.ravel(), out.ravel()
    for i in range(xf.size):
        of[i] = L.tso_float_to_i8(float(xf[i]))
    return out


def att_dot_scale(d):
    return np.float32(lib().tso_att_dot_scale(int(d)))


def quantize_rows(dtype, x, n_heads):
    """x: [n_rows, n_heads*d] float32 (or uint16 holding bf16 bits) -> (q uint8 [n_rows, H*d], scale f32 [H, n_rows])."""
    L = lib()
    n_rows, hd = x.shape
    d = hd // n_heads
    q = np.empty((n_rows, hd), dtype=np.uint8)
    scale = np.empty((n_heads, n_rows), dtype=np.float32)
    if x.dtype == np.uint16:
        x = np.ascontiguousarray(x)
        L.tso_quantize_rows_bf16(dtype, _p(x), hd, n_rows, n_heads, d, _p(q), hd, _p(scale), n_rows)
    else:
        x = _c_arr(x, np.float32)
        L.tso_quantize_rows(dtype, _p(x), hd, n_rows, n_heads, d, _p(q), hd, _p(scale), n_rows)
    return q, scale


def float_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    return r


def bf16_bits_to_float(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---- masks -----------------------------------------------------------------------------------
def fill_rope(width, max_len):
    L = lib()
    rope = np.empty((max_len, width), dtype=np.float32)
    L.tso_fill_rope(int(width), ctypes.c_int64(max_len), _p(rope))
    return rope


def apply_rope(rope_row, rotate_dir, vec, head_size):
    L = lib()
    v = np.array(vec, dtype=np.float32, copy=True)
    r = _c_arr(rope_row, np.float32)
    L.tso_apply_rope(_p(r), ctypes.c_float(rotate_dir), int(v.size), int(head_size), _p(v))
    return v


def rope_normalize_rows(dtype, x, n_heads, pos=None, rope=None, rotate_dir=1.0, vec_scale=1.0 / 24, scale_mult=1.0):
    """x: [n_rows, H*d] float32 or int32 -> (q uint8 [n_rows, H*d], scale f32 [H, n_rows])."""
    L = lib()
    is_i32 = x.dtype == np.int32
    x = _c_arr(x, np.int32 if is_i32 else np.float32)
    n_rows, hd = x.shape
    d = hd // n_heads
    q = np.empty((n_rows, hd), dtype=np.uint8)
    scale = np.empty((n_heads, n_rows), dtype=np.float32)
    ps = None if pos is None else _c_arr(pos, np.int32)
    rp = None if rope is None else _c_arr(rope, np.float32)
    L.tso_rope_normalize_rows(int(dtype), _p(x), int(is_i32), ctypes.c_int64(hd), ctypes.c_int64(n_rows), _p(ps), _p(rp),
                              ctypes.c_float(rotate_dir), int(n_heads), int(d), ctypes.c_float(vec_scale),
                              ctypes.c_float(scale_mult), _p(q), ctypes.c_int64(hd), _p(scale), ctypes.c_int64(n_rows))
    return q, scale


def kv_product(k, val, n_heads, rep=4, mult=1.0):
    """k: int8 (as uint8 or int8) [n_rows, H*d]; val: float32 [n_rows, H*d] -> int8 [n_rows, H*d*rep]."""
    L = lib()
    k = _c_arr(np.asarray(k).view(np.int8), np.int8)
    val = _c_arr(val, np.float32)
    n, hd = k.shape
    kv = np.empty((n, hd * rep), dtype=np.int8)
    L.tso_kv_product(_p(k), ctypes.c_int64(hd), _p(val), ctypes.c_int64(hd), ctypes.c_int64(n), int(n_heads), int(hd // n_heads),
                     int(rep), ctypes.c_float(mult), _p(kv), ctypes.c_int64(hd * rep))
    return kv


def matmul_i8(a, w, mode=0, scale=1.0, out=None):
    """a: int8 [m, k], w: int8 [n, k] -> [m, n]: int32 sums (mode 0), float32 sums * scale (1), out += sums * scale (2)."""
    L = lib()
    a = _c_arr(np.asarray(a).view(np.int8), np.int8)
    w = _c_arr(np.asarray(w).view(np.int8), np.int8)
    m, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k and k % 64 == 0
    if mode == 2:
        out = _c_arr(out, np.float32).copy()
    else:
        out = np.empty((m, n), dtype=np.int32 if mode == 0 else np.float32)
    L.tso_matmul_i8(_p(a), ctypes.c_int64(k), _p(w), ctypes.c_int64(k), ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int64(k),
                    int(mode), ctypes.c_float(scale), _p(out), ctypes.c_int64(n))
    return out


class LayerParams(ctypes.Structure):
    _fields_ = [("dim", ctypes.c_int), ("head_count", ctypes.c_int), ("head_dim", ctypes.c_int), ("relu_dim", ctypes.c_int),
                ("qk", ctypes.c_void_p), ("qv", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
                ("combiner", ctypes.c_void_p), ("expand", ctypes.c_void_p), ("contract", ctypes.c_void_p),
                ("qv_scale", ctypes.c_float), ("combiner_scale", ctypes.c_float), ("contract_scale", ctypes.c_float),
                ("attention_width", ctypes.c_int64), ("alibi_slope", ctypes.c_float)]


def add_lookup_product(mats, scales, width, slope, head_count, head_dim, t, rope, state, k_cache, v_cache, k_scale_cache, cache_len):
    """AddLookupProduct (cpu_infer.cpp:465-527) for one token per sequence.  mats: dict of int8 arrays qk, qv, k, v
    [H*d, dim], combiner [dim, 4*H*d], expand [relu, dim], contract [dim, relu]; scales: (qv, combiner, contract).
    Caches planar [n_seq, H, max_len, d] (uint8) and [n_seq, H, max_len] (float32), cache_len int32 [n_seq]: all updated
    in place.  Returns (new state, attention output)."""
    L = lib()
    keep = {k: _c_arr(np.asarray(v).view(np.int8), np.int8) for k, v in mats.items()}
    n_seq, dim = state.shape
    P = LayerParams()
    P.dim, P.head_count, P.head_dim, P.relu_dim = dim, head_count, head_dim, keep["expand"].shape[0]
    for name in ("qk", "qv", "k", "v", "combiner", "expand", "contract"):
        setattr(P, name, keep[name].ctypes.data)
    P.qv_scale, P.combiner_scale, P.contract_scale = scales
    P.attention_width, P.alibi_slope = int(width), float(slope)
    out = _c_arr(state, np.float32).copy()
    val = np.zeros((n_seq, head_count * head_dim), dtype=np.float32)
    t = _c_arr(t, np.int32)
    rope = _c_arr(rope, np.float32)
    for a, dt in ((k_cache, np.uint8), (v_cache, np.uint8), (k_scale_cache, np.float32), (cache_len, np.int32)):
        assert a.dtype == dt and a.flags["C_CONTIGUOUS"]
    max_len = k_cache.shape[2]
    L.tso_add_lookup_product(ctypes.byref(P), ctypes.c_int64(n_seq), _p(t), _p(rope), _p(out), _p(k_cache), _p(v_cache),
                             ctypes.c_int64(head_count * max_len * head_dim), ctypes.c_int64(max_len * head_dim), ctypes.c_int64(head_dim),
                             _p(k_scale_cache), ctypes.c_int64(head_count * max_len), ctypes.c_int64(max_len), _p(cache_len), int(max_len),
                             _p(val), 2)
    return out, val


def embed_rows(labels, embed, scale):
    """labels int32 [n_rows] or [n_rows, L]; embed int8 [n_labels, dim] -> float32 [n_rows, dim]."""
    L = lib()
    labels = _c_arr(np.asarray(labels).reshape(len(labels), -1), np.int32)
    embed = _c_arr(np.asarray(embed).view(np.int8), np.int8)
    n_rows, per_row = labels.shape
    n_labels, dim = embed.shape
    out = np.empty((n_rows, dim), dtype=np.float32)
    L.tso_embed_rows(ctypes.c_int64(n_rows), int(dim), _p(labels), int(per_row), _p(embed), ctypes.c_int64(n_labels), ctypes.c_float(scale), _p(out))
    return out


def softmax_rows(vec, scale, bias=None, exp2_mode=0):
    """vec int32 [n_rows, n] -> (prob float32 [n_rows, n], argmax int32 [n_rows])."""
    L = lib()
    vec = _c_arr(vec, np.int32)
    n_rows, n = vec.shape
    b = None if bias is None else _c_arr(bias, np.float32)
    prob = np.empty((n_rows, n), dtype=np.float32)
    arg = np.empty(n_rows, dtype=np.int32)
    L.tso_softmax_rows(ctypes.c_int64(n_rows), ctypes.c_int64(n), _p(vec), ctypes.c_float(scale), _p(b), int(exp2_mode), _p(prob), _p(arg))
    return prob, arg


def mix32(seed, index):
    L = lib()
    L.tso_mix32.restype = ctypes.c_uint32
    return int(L.tso_mix32(ctypes.c_uint64(seed), ctypes.c_uint64(index)))


def sample_rows(prob, temperature, rnd=None, seed=0, offset=0):
    """prob float32 [n_rows, n] -> the Gumbel-max choice per row, int32 [n_rows]; rnd: uint32 words [n_rows, n] or None
    (the counter generator on seed and offset)."""
    L = lib()
    prob = _c_arr(prob, np.float32)
    n_rows, n = prob.shape
    r = None if rnd is None else _c_arr(rnd, np.uint32)
    choice = np.empty(n_rows, dtype=np.int32)
    L.tso_sample_rows(ctypes.c_int64(n_rows), ctypes.c_int64(n), _p(prob), ctypes.c_int64(n), ctypes.c_float(temperature), _p(r),
                      ctypes.c_int64(n), ctypes.c_uint64(seed), ctypes.c_uint64(offset), _p(choice))
    return choice


def make_spans(seq_lens, window, doc_start_flag=None):
    L = lib()
    off = np.zeros(len(seq_lens) + 1, dtype=np.int64)
    off[1:] = np.cumsum(seq_lens)
    n = int(off[-1])
    st = np.empty(n, dtype=np.int32)
    fi = np.empty(n, dtype=np.int32)
    flag = None if doc_start_flag is None else _c_arr(doc_start_flag, np.uint8)
    L.tso_make_spans(len(seq_lens), _p(off), _p(flag), int(window), _p(st), _p(fi))
    return st, fi


def init_alibi(depth, wide):
    L = lib()
    w = np.zeros(depth + 2, dtype=np.int64)
    s = np.zeros(depth + 2, dtype=np.float32)
    n = L.tso_init_alibi(int(depth), int(wide), depth + 2, _p(w), _p(s))
    return w[:n].copy(), s[:n].copy()


# ---- dots ------------------------------------------------------------------------------------
def dot_i8(a, b, simd=False):
    L = lib()
    a = _c_arr(a, np.int8)
    b = _c_arr(b, np.int8)
    f = L.tso_dot_i8_simd if simd else L.tso_dot_i8
    return int(f(_p(a), _p(b), a.size))


def dot_e4m3(a, b):
    L = lib()
    a = _c_arr(a, np.uint8)
    b = _c_arr(b, np.uint8)
    return np.float32(L.tso_dot_e4m3(_p(a), _p(b), a.size))


def qk_accum(dtype, q, k, head, d, from0, n_from, to0, n_to):
    L = lib()
    q = _c_arr(q, np.uint8)
    k = _c_arr(k, np.uint8)
    acc = np.empty((n_from, n_to), dtype=np.int32 if dtype == I8 else np.float32)
    L.tso_qk_accum(dtype, _p(q), q.shape[1], _p(k), k.shape[1], head, d, from0, n_from, to0, n_to, _p(acc))
    return acc


# ---- attention --------------------------------------------------------------------------------
def prefill_f32(qk, qv, v, n_heads, span_ptr, spans, slope):
    L = lib()
    qk = _c_arr(qk, np.float32)
    qv = _c_arr(qv, np.float32)
    v = _c_arr(v, np.float32)
    n = qk.shape[0]
    q_dim = qk.shape[1] // n_heads
    tt_dim = v.shape[1] // n_heads
    span_ptr = _c_arr(span_ptr, np.int32)
    spans = _c_arr(spans, np.int32)
    out = np.empty((n, n_heads * tt_dim), dtype=np.float32)
    sw = np.empty((n_heads, n), dtype=np.float32)
    mx = np.empty((n_heads, n), dtype=np.float32)
    L.tso_prefill_f32(n, n_heads, q_dim, tt_dim, _p(qk), _p(qv), _p(v), _p(span_ptr), _p(spans),
                      float(slope), _p(out), _p(sw), _p(mx))
    return out, sw, mx


def _scale_args(s, default):
    if s is None:
        return None, float(default)
    if np.isscalar(s):
        return None, float(s)
    return _c_arr(s, np.float32), 0.0


def prefill_q8(dtype, q, k, v, n_heads, q_scale, k_scale, v_scale, span_start, span_finish, slope,
               want_swl=False, n_threads=0):
    """q,k,v: uint8 [n_tokens, H*d]; scales f32 [H, n_tokens] or python scalars."""
    L = lib()
    q = _c_arr(q, np.uint8)
    k = _c_arr(k, np.uint8)
    v = _c_arr(v, np.uint8)
    n, hd = q.shape
    d = hd // n_heads
    qs, qc = _scale_args(q_scale, 1.0)
    ks, kc = _scale_args(k_scale, 1.0)
    vs, vc = _scale_args(v_scale, 1.0)
    st = _c_arr(span_start, np.int32)
    fi = _c_arr(span_finish, np.int32)
    out = np.empty((n, hd), dtype=np.float32)
    swl = np.empty((n_heads, n), dtype=np.float32) if want_swl else None
    if n_threads <= 0:
        n_threads = L.tso_max_threads()
    L.tso_prefill_q8(dtype, n, n_heads, d, _p(q), _p(k), _p(v), hd, _p(qs), _p(ks), _p(vs), n,
                     qc, kc, vc, _p(st), _p(fi), float(slope), _p(out), hd, _p(swl), n_threads)
    return (out, swl) if want_swl else out


def decode(dtype, q, q_scale, k_cache, v_cache, k_scale, v_scale, cache_len, window, slope,
           exp2_mode=0, use_simd=False, want_acc=False, n_threads=0):
    """Planar cache: k_cache, v_cache uint8 [B, H, L, d]; k_scale, v_scale f32 [B, H, L] (or scalars);
    q uint8 [B, H*d]; q_scale f32 [B, H] or scalar; cache_len int32 [B]."""
    L = lib()
    k_cache = _c_arr(k_cache, np.uint8)
    v_cache = _c_arr(v_cache, np.uint8)
    B, H, Lmax, d = k_cache.shape
    q = _c_arr(q, np.uint8)
    qs, qc = _scale_args(q_scale, 1.0)
    ks, kc = _scale_args(k_scale, 1.0)
    vs, vc = _scale_args(v_scale, 1.0)
    cl = _c_arr(cache_len, np.int32)
    out = np.empty((B, H * d), dtype=np.float32)
    acc = None
    if want_acc:
        acc = np.zeros((B, H, Lmax), dtype=np.int32 if dtype == I8 else np.float32)
    if n_threads <= 0:
        n_threads = L.tso_max_threads()
    L.tso_decode(dtype, B, H, d, _p(q), _p(qs), qc, _p(k_cache), _p(v_cache), H * Lmax * d, Lmax * d, d,
                 _p(ks), _p(vs), H * Lmax, Lmax, kc, vc, _p(cl), int(window), float(slope),
                 int(exp2_mode), int(bool(use_simd)), _p(out), _p(acc), Lmax, n_threads)
    return (out, acc) if want_acc else out


def softmax_buf(logits, exp2_mode):
    L = lib()
    x = _c_arr(logits, np.float32)
    w = np.empty_like(x)
    scale = L.tso_softmax_buf(_p(x), x.size, int(exp2_mode), _p(w))
    return w, np.float32(scale)


def simd_level():
    return lib().tso_simd_level()


def max_threads():
    return lib().tso_max_threads()
