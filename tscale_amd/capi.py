"""ctypes binding of libtsattn.so (the C ABI declared in include/tsattn.h).

This module is plumbing: it loads the HIP library built in-tree and mirrors the C structs.  It has
no CPU fallback; if the library is missing or a call fails, it raises.
"""
import ctypes
import os

_c = ctypes
_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtsattn.so")

I8, E4M3 = 0, 1
OUT_F32, OUT_F16 = 0, 1
SRC_F32, SRC_BF16, SRC_I32 = 0, 1, 2
MM_I32, MM_F32, MM_ADD_SCALED, MM_I32_PLANES = 0, 1, 2, 3
Q_8BIT, Q_BF16 = 0, 1
SPAN_TILE_INTS = 32
PREFILL_LONG_SPAN = 6144   # TSATTN_PREFILL_LONG_SPAN: span_len_hint from which tsattn_prefill uses a workspace

STATUS_NAMES = {0: "OK", 1: "BAD_ARG", 2: "UNSUPPORTED", 3: "HIP", 4: "SCRATCH"}


class TsattnError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"tsattn error {code} ({STATUS_NAMES.get(code, '?')}): {text}")
        self.code = code


class Config(_c.Structure):
    _fields_ = [("device", _c.c_int), ("max_seqs", _c.c_int), ("max_heads", _c.c_int),
                ("max_head_dim", _c.c_int), ("max_splits", _c.c_int)]


class PrefillArgs(_c.Structure):
    _fields_ = [
        ("dtype", _c.c_int), ("out_dtype", _c.c_int), ("n_tokens", _c.c_int64), ("n_heads", _c.c_int),
        ("head_dim", _c.c_int), ("q", _c.c_void_p), ("k", _c.c_void_p), ("v", _c.c_void_p),
        ("q_pitch", _c.c_int64), ("k_pitch", _c.c_int64), ("v_pitch", _c.c_int64),
        ("q_scale", _c.c_void_p), ("k_scale", _c.c_void_p), ("v_scale", _c.c_void_p),
        ("scale_pitch", _c.c_int64), ("q_scale_const", _c.c_float), ("k_scale_const", _c.c_float),
        ("v_scale_const", _c.c_float), ("k_global_scale", _c.c_void_p), ("span_start", _c.c_void_p),
        ("span_finish", _c.c_void_p), ("alibi_slope", _c.c_float), ("out", _c.c_void_p),
        ("out_pitch", _c.c_int64), ("sum_weight_log", _c.c_void_p), ("debug_qk_acc", _c.c_void_p),
        ("debug_pitch", _c.c_int64), ("span_tiles", _c.c_void_p), ("causal_period", _c.c_int64),
        ("kv_k", _c.c_void_p), ("kv_k_pitch", _c.c_int64), ("kv_out", _c.c_void_p), ("kv_out_pitch", _c.c_int64),
        ("kv_rep", _c.c_int), ("kv_mult", _c.c_float),
        ("workspace", _c.c_void_p), ("workspace_bytes", _c.c_int64), ("span_len_hint", _c.c_int64),
        ("n_span_parts", _c.c_int), ("span_part_stride", _c.c_int64),
    ]


class DecodeArgs(_c.Structure):
    _fields_ = [
        ("dtype", _c.c_int), ("q_dtype", _c.c_int), ("n_seqs", _c.c_int), ("n_heads", _c.c_int),
        ("head_dim", _c.c_int), ("q", _c.c_void_p), ("q_pitch", _c.c_int64), ("q_scale", _c.c_void_p),
        ("q_scale_const", _c.c_float), ("k_cache", _c.c_void_p), ("v_cache", _c.c_void_p),
        ("seq_stride", _c.c_int64), ("head_stride", _c.c_int64), ("tok_stride", _c.c_int64),
        ("k_scale", _c.c_void_p), ("v_scale", _c.c_void_p), ("s_seq_stride", _c.c_int64),
        ("s_head_stride", _c.c_int64), ("k_scale_const", _c.c_float), ("v_scale_const", _c.c_float),
        ("cache_len", _c.c_void_p), ("max_len", _c.c_int), ("window", _c.c_int64),
        ("alibi_slope", _c.c_float), ("out", _c.c_void_p), ("n_splits", _c.c_int),
        ("debug_qk_acc", _c.c_void_p), ("debug_pitch", _c.c_int64), ("k_new", _c.c_void_p), ("v_new", _c.c_void_p),
        ("new_pitch", _c.c_int64), ("k_scale_new", _c.c_void_p), ("v_scale_new", _c.c_void_p),
        ("kv_k", _c.c_void_p), ("kv_k_pitch", _c.c_int64), ("kv_out", _c.c_void_p), ("kv_out_pitch", _c.c_int64),
        ("kv_rep", _c.c_int), ("kv_mult", _c.c_float),
    ]


class AppendArgs(_c.Structure):
    _fields_ = [
        ("n_seqs", _c.c_int), ("n_heads", _c.c_int), ("head_dim", _c.c_int), ("k_new", _c.c_void_p),
        ("v_new", _c.c_void_p), ("new_pitch", _c.c_int64), ("k_scale_new", _c.c_void_p),
        ("v_scale_new", _c.c_void_p), ("k_cache", _c.c_void_p), ("v_cache", _c.c_void_p),
        ("seq_stride", _c.c_int64), ("head_stride", _c.c_int64), ("tok_stride", _c.c_int64),
        ("k_scale", _c.c_void_p), ("v_scale", _c.c_void_p), ("s_seq_stride", _c.c_int64),
        ("s_head_stride", _c.c_int64), ("cache_len", _c.c_void_p), ("max_len", _c.c_int),
    ]


class ProduceArgs(_c.Structure):
    _fields_ = [
        ("src_dtype", _c.c_int), ("dst_dtype", _c.c_int), ("n_rows", _c.c_int64), ("n_heads", _c.c_int),
        ("head_dim", _c.c_int), ("src", _c.c_void_p), ("src_pitch", _c.c_int64), ("pos", _c.c_void_p),
        ("rope", _c.c_void_p), ("rope_len", _c.c_int64), ("rotate_dir", _c.c_float), ("vec_scale", _c.c_float),
        ("scale_mult", _c.c_float), ("dst", _c.c_void_p), ("dst_pitch", _c.c_int64), ("scale", _c.c_void_p),
        ("scale_pitch", _c.c_int64), ("scale_row_stride", _c.c_int64), ("relu", _c.c_int),
        ("src_planes", _c.c_int), ("src_plane_stride", _c.c_int64), ("rope_heads", _c.c_int), ("scale_head_begin", _c.c_int),
        ("scale_head_count", _c.c_int), ("resid", _c.c_void_p), ("resid_pitch", _c.c_int64), ("resid_scale", _c.c_float),
    ]


class MatmulArgs(_c.Structure):
    _fields_ = [
        ("m", _c.c_int64), ("n", _c.c_int64), ("k", _c.c_int64), ("a", _c.c_void_p), ("a_pitch", _c.c_int64),
        ("w", _c.c_void_p), ("w_pitch", _c.c_int64), ("mode", _c.c_int), ("scale", _c.c_float), ("out", _c.c_void_p),
        ("out_pitch", _c.c_int64), ("workspace", _c.c_void_p), ("workspace_bytes", _c.c_int64), ("planes_out", _c.POINTER(_c.c_int)),
        ("epilogue", _c.c_void_p),
    ]


class FillArgs(_c.Structure):
    _fields_ = [
        ("n_seqs", _c.c_int), ("n_heads", _c.c_int), ("head_dim", _c.c_int), ("n_tokens", _c.c_int64),
        ("seq_offset", _c.c_void_p), ("k", _c.c_void_p), ("v", _c.c_void_p), ("pitch", _c.c_int64),
        ("k_scale", _c.c_void_p), ("v_scale", _c.c_void_p), ("scale_pitch", _c.c_int64),
        ("k_cache", _c.c_void_p), ("v_cache", _c.c_void_p), ("seq_stride", _c.c_int64),
        ("head_stride", _c.c_int64), ("tok_stride", _c.c_int64), ("k_scale_cache", _c.c_void_p),
        ("v_scale_cache", _c.c_void_p), ("s_seq_stride", _c.c_int64), ("s_head_stride", _c.c_int64),
        ("cache_len", _c.c_void_p), ("max_len", _c.c_int),
    ]


class MergeArgs(_c.Structure):
    _fields_ = [
        ("n_parts", _c.c_int), ("n_tokens", _c.c_int64), ("n_heads", _c.c_int), ("head_dim", _c.c_int),
        ("part_out", _c.c_void_p), ("part_out_pitch", _c.c_int64), ("part_out_stride", _c.c_int64),
        ("part_swl", _c.c_void_p), ("scale_pitch", _c.c_int64), ("part_swl_stride", _c.c_int64),
        ("out_dtype", _c.c_int), ("out", _c.c_void_p), ("out_pitch", _c.c_int64), ("sum_weight_log", _c.c_void_p),
    ]


EXPORTS = ["tsattn_scratch_bytes", "tsattn_create", "tsattn_destroy", "tsattn_last_error", "tsattn_prefill", "tsattn_prefill_workspace_bytes",
           "tsattn_decode", "tsattn_decode_static", "tsattn_cache_append", "tsattn_cache_fill", "tsattn_merge_lookups", "tsattn_span_tiles_count", "tsattn_build_span_tiles", "tsattn_rope_normalize_rows", "tsattn_fill_rope_table", "tsattn_kv_product", "tsattn_matmul_i8", "tsattn_embed_rows", "tsattn_softmax_rows", "tsattn_sample_rows", "tsattn_quantize_rows", "tsattn_build_spans", "tsattn_debug_read_counters", "tsattn_version"]

_lib = None


def load():
    """Load the in-tree HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `make -C tscale_amd/csrc` (hipcc, gfx950). "
                "There is no CPU fallback.")
        L = ctypes.CDLL(LIB_PATH)
        L.tsattn_scratch_bytes.restype = _c.c_size_t
        L.tsattn_scratch_bytes.argtypes = [_c.POINTER(Config)]
        L.tsattn_create.restype = _c.c_int
        L.tsattn_create.argtypes = [_c.POINTER(Config), _c.POINTER(_c.c_void_p)]
        L.tsattn_destroy.restype = _c.c_int
        L.tsattn_destroy.argtypes = [_c.c_void_p]
        L.tsattn_last_error.restype = _c.c_char_p
        L.tsattn_version.restype = _c.c_char_p
        L.tsattn_prefill.restype = _c.c_int
        L.tsattn_prefill.argtypes = [_c.c_void_p, _c.POINTER(PrefillArgs), _c.c_void_p]
        L.tsattn_prefill_workspace_bytes.restype = _c.c_size_t
        L.tsattn_prefill_workspace_bytes.argtypes = [_c.c_int64, _c.c_int, _c.c_int]
        L.tsattn_decode.restype = _c.c_int
        L.tsattn_decode.argtypes = [_c.c_void_p, _c.POINTER(DecodeArgs), _c.c_void_p]
        L.tsattn_debug_read_counters.restype = _c.c_int
        L.tsattn_debug_read_counters.argtypes = [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p]
        L.tsattn_decode_static.restype = _c.c_int
        L.tsattn_decode_static.argtypes = [_c.POINTER(DecodeArgs), _c.c_void_p]
        L.tsattn_cache_append.restype = _c.c_int
        L.tsattn_cache_append.argtypes = [_c.c_void_p, _c.POINTER(AppendArgs), _c.c_void_p]
        L.tsattn_cache_fill.restype = _c.c_int
        L.tsattn_cache_fill.argtypes = [_c.c_void_p, _c.POINTER(FillArgs), _c.c_void_p]
        L.tsattn_merge_lookups.restype = _c.c_int
        L.tsattn_merge_lookups.argtypes = [_c.c_void_p, _c.POINTER(MergeArgs), _c.c_void_p]
        L.tsattn_span_tiles_count.restype = _c.c_int64
        L.tsattn_span_tiles_count.argtypes = [_c.c_int64]
        L.tsattn_build_span_tiles.restype = _c.c_int
        L.tsattn_build_span_tiles.argtypes = [_c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p]
        L.tsattn_rope_normalize_rows.restype = _c.c_int
        L.tsattn_rope_normalize_rows.argtypes = [_c.c_void_p, _c.POINTER(ProduceArgs), _c.c_void_p]
        L.tsattn_fill_rope_table.restype = None
        L.tsattn_fill_rope_table.argtypes = [_c.c_int, _c.c_int64, _c.c_void_p]
        L.tsattn_kv_product.restype = _c.c_int
        L.tsattn_kv_product.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int,
                                        _c.c_void_p, _c.c_int64, _c.c_float, _c.c_void_p, _c.c_int64, _c.c_void_p]
        L.tsattn_matmul_i8.restype = _c.c_int
        L.tsattn_matmul_i8.argtypes = [_c.c_void_p, _c.POINTER(MatmulArgs), _c.c_void_p]
        L.tsattn_embed_rows.restype = _c.c_int
        L.tsattn_embed_rows.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int64,
                                        _c.c_float, _c.c_void_p, _c.c_int64, _c.c_void_p]
        L.tsattn_softmax_rows.restype = _c.c_int
        L.tsattn_softmax_rows.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_float,
                                          _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p]
        L.tsattn_sample_rows.restype = _c.c_int
        L.tsattn_sample_rows.argtypes = [_c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_int64, _c.c_float, _c.c_void_p, _c.c_int64,
                                         _c.c_uint64, _c.c_uint64, _c.c_void_p, _c.c_void_p]
        L.tsattn_quantize_rows.restype = _c.c_int
        L.tsattn_quantize_rows.argtypes = [_c.c_void_p, _c.c_int, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int64,
                                           _c.c_int, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int64,
                                           _c.c_void_p]
        L.tsattn_build_spans.restype = _c.c_int
        L.tsattn_build_spans.argtypes = [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int64,
                                         _c.c_void_p, _c.c_void_p, _c.c_void_p]
        _lib = L
    return _lib


def check(code):
    if code != 0:
        raise TsattnError(code, load().tsattn_last_error().decode())
