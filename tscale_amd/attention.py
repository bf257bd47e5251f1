"""Host-side mirror of the reference's attention call sites on top of the C ABI.

`AttentionContext.compute_val_lookup` has the argument meaning of
TAttentionComputer::ComputeValLookup (gpt/compute/gpt_cpu.cpp:391-441) / the Fp8Att launch
(gpt/compute/gpt_cuda.cu:503-507); `AttentionContext.compute_val_lookup_decode` that of
ComputeValLookup in gpt/train/cpu_infer.cpp:413-460 and `KVCache.add_vectors` that of
TAttentionVecHistory::AddVectors (:403-408).  torch tensors are used for device memory only; all
arithmetic happens in libtsattn.so.  There is no fallback path: a missing library raises.
"""
import ctypes

import numpy as np
import torch

from . import capi


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _scale_arg(s):
    """tensor -> (pointer, 0.0); python number -> (None, value)."""
    if isinstance(s, torch.Tensor):
        assert s.dtype == torch.float32 and s.is_cuda and s.is_contiguous()
        return _ptr(s), 0.0
    return None, float(s)


def alibi_layer_schedule(depth, wide_window):
    """Per-layer (attention width, ALiBi slope) of a TScale model of `depth` layers: the ALIBI_V3 rule of
    InitAlibi (gpt/model_params/model_dim.cpp:55-97): max(1, groups/6) leading pairs of width-1 layers,
    then pairs of (64, slope 0.5) and (wide, slope 0); a one-layer model is (wide, 0.1)."""
    if depth == 1:
        return [(wide_window, 0.1)]
    groups = (depth + 1) // 2
    w1 = max(1, groups // 6)
    out = []
    for _ in range(w1):
        out += [(1, 0.0), (1, 0.0)]
    for _ in range(w1, groups):
        out += [(64, 0.5), (wide_window, 0.0)]
    return out


class AttentionContext:
    """One per device, like the reference's per-device compute context (gpt_cuda.cu:1478-1573)."""

    def __init__(self, device=0, max_seqs=64, max_heads=16, max_head_dim=128, max_splits=32):
        self.lib = capi.load()
        if not torch.cuda.is_available():
            raise RuntimeError("tscale_amd needs a HIP device; there is no CPU path")
        cfg = capi.Config(device, max_seqs, max_heads, max_head_dim, max_splits)
        h = ctypes.c_void_p()
        capi.check(self.lib.tsattn_create(ctypes.byref(cfg), ctypes.byref(h)))
        self.handle = h
        self.device = torch.device("cuda", device)
        self._workspace = None  # scratch of the long-span prefill kernel, grown on demand

    def close(self):
        if self.handle:
            self.lib.tsattn_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- producers of the path's inputs -------------------------------------------------------
    def quantize_rows(self, x, n_heads, dtype):
        """x: [n_rows, n_heads*d] float32 or bfloat16 -> (uint8 [n_rows, n_heads*d], f32 [n_heads, n_rows])."""
        assert x.is_cuda and x.is_contiguous() and x.dim() == 2
        n_rows, hd = x.shape
        src = capi.SRC_F32 if x.dtype == torch.float32 else capi.SRC_BF16
        assert x.dtype in (torch.float32, torch.bfloat16)
        q = torch.empty((n_rows, hd), dtype=torch.uint8, device=x.device)
        scale = torch.empty((n_heads, n_rows), dtype=torch.float32, device=x.device)
        capi.check(self.lib.tsattn_quantize_rows(self.handle, src, dtype, _ptr(x), hd * x.element_size(), n_rows,
                                                 n_heads, hd // n_heads, _ptr(q), hd, _ptr(scale), n_rows,
                                                 _stream_ptr()))
        return q, scale

    def fill_rope_table(self, head_dim, max_len):
        """The table of FillRopeBuf (gpt/att/rope.cpp:4-24), computed on the host by the library, on the device."""
        host = torch.empty((max_len, head_dim), dtype=torch.float32)
        self.lib.tsattn_fill_rope_table(head_dim, max_len, ctypes.c_void_p(host.data_ptr()))
        return host.to(self.device)

    def _produce_args(self, n_rows, hd, device, n_heads, dtype, pos, rope, rotate_dir, vec_scale, scale_mult, row_major_scale, relu,
                      rope_heads, scale_heads, resid, resid_scale):
        """The producer's arguments (without its source) and its two results."""
        q = torch.empty((n_rows, hd), dtype=torch.uint8, device=device)
        n_scale = n_heads if scale_heads is None else scale_heads[1]
        scale = torch.empty((n_rows, n_scale) if row_major_scale else (n_scale, n_rows), dtype=torch.float32, device=device)
        a = capi.ProduceArgs()
        a.dst_dtype = dtype
        a.n_rows, a.n_heads, a.head_dim = n_rows, n_heads, hd // n_heads
        a.pos, a.rope = _ptr(pos), _ptr(rope)
        a.rope_len = 0 if rope is None else rope.shape[0]
        a.rope_heads = int(rope_heads)
        a.rotate_dir, a.vec_scale, a.scale_mult = float(rotate_dir), float(vec_scale), float(scale_mult)
        a.dst, a.dst_pitch = _ptr(q), hd
        a.scale, a.scale_pitch = _ptr(scale), (1 if row_major_scale else n_rows)
        a.scale_row_stride = n_scale if row_major_scale else 1
        if scale_heads is not None:
            a.scale_head_begin, a.scale_head_count = int(scale_heads[0]), int(scale_heads[1])
        a.relu = int(bool(relu))
        if resid is not None:
            assert resid.dtype == torch.float32 and resid.shape == (n_rows, hd) and resid.stride(1) == 1
            a.resid, a.resid_pitch, a.resid_scale = _ptr(resid), resid.stride(0), float(resid_scale)
        return a, q, scale

    def rope_normalize_rows(self, x, n_heads, dtype, pos=None, rope=None, rotate_dir=1.0, vec_scale=1.0 / 24,
                            scale_mult=1.0, row_major_scale=False, relu=False, rope_heads=0, scale_heads=None,
                            resid=None, resid_scale=1.0):
        """ApplyRope + NormalizeState of the reference's inference path (cpu_infer.cpp:486-499): x [n_rows, H*d]
        float32 or int32 -> (uint8 [n_rows, H*d], f32 scale [H, n_rows], or [n_rows, H] with row_major_scale: what
        the cache append reads); pos int32 [n_rows] or None (no rotation); relu: negative results become 0 (:520-524).
        x may be int32 [planes, n_rows, H*d]: the parts of a split-K product, summed on the fly.  rope_heads: only the
        heads below it are rotated.  scale_heads = (begin, count): scales only for those heads.  resid (f32
        [n_rows, H*d]): resid += x * resid_scale first, in place, and the updated rows are normalised."""
        assert x.is_cuda and x.is_contiguous() and x.dtype in (torch.float32, torch.int32)
        planes = 1
        if x.dim() == 3:
            assert x.dtype == torch.int32
            planes = x.shape[0]
        n_rows, hd = x.shape[-2:]
        a, q, scale = self._produce_args(n_rows, hd, x.device, n_heads, dtype, pos, rope, rotate_dir, vec_scale, scale_mult, row_major_scale,
                                         relu, rope_heads, scale_heads, resid, resid_scale)
        a.src_dtype = capi.SRC_F32 if x.dtype == torch.float32 else capi.SRC_I32
        a.src, a.src_pitch = _ptr(x), hd
        a.src_planes, a.src_plane_stride = planes, n_rows * hd
        capi.check(self.lib.tsattn_rope_normalize_rows(self.handle, ctypes.byref(a), _stream_ptr()))
        return q, scale

    def matmul_normalize(self, a, w, n_heads, dtype, scratch=None, **producer):
        """MulForward followed by rope_normalize_rows on its int32 result, as one library call: the projection with its
        normalising epilogue.  Large products with an int8 result never write the int32 sums (the product's kernel
        normalises its own tiles).  a uint8 [m, k], w uint8 [n, k]; scratch: int32 room for 16 * m * n sums (m <= 128) or
        m * n, made here if not given; producer: rope_normalize_rows' keyword arguments.  Returns (uint8 [m, n], scale)
        like rope_normalize_rows."""
        m, k = a.shape
        n = w.shape[0]
        assert w.shape[1] == k and a.stride(1) == 1 and w.stride(1) == 1
        room = (16 if m <= 128 else 1) * m * n
        if scratch is None:
            scratch = torch.empty(room, dtype=torch.int32, device=a.device)
        assert scratch.is_contiguous() and scratch.dtype == torch.int32 and scratch.numel() >= room
        kw = dict(pos=None, rope=None, rotate_dir=1.0, vec_scale=1.0 / 24, scale_mult=1.0, row_major_scale=False, relu=False, rope_heads=0,
                  scale_heads=None, resid=None, resid_scale=1.0)
        kw.update(producer)
        ep, q, scale = self._produce_args(m, n, a.device, n_heads, dtype, kw["pos"], kw["rope"], kw["rotate_dir"], kw["vec_scale"], kw["scale_mult"],
                                          kw["row_major_scale"], kw["relu"], kw["rope_heads"], kw["scale_heads"], kw["resid"], kw["resid_scale"])
        args = capi.MatmulArgs()
        args.m, args.n, args.k = m, n, k
        args.a, args.a_pitch = _ptr(a), a.stride(0)
        args.w, args.w_pitch = _ptr(w), w.stride(0)
        args.mode, args.scale = capi.MM_I32_PLANES, 1.0
        args.out, args.out_pitch = _ptr(scratch), n
        planes = ctypes.c_int(0)
        args.planes_out = ctypes.pointer(planes)
        args.epilogue = ctypes.cast(ctypes.pointer(ep), ctypes.c_void_p)
        capi.check(self.lib.tsattn_matmul_i8(self.handle, ctypes.byref(args), _stream_ptr()))
        return q, scale

    def kv_product(self, k, value, n_heads, rep=4, mult=1.0):
        """KVProduct (cpu_infer.cpp:320-337): k uint8 (int8 bytes) [n, H*d], value f32/f16 [n, H*d] -> uint8 [n, H*d*rep]."""
        n, hd = k.shape
        assert value.shape == k.shape and value.is_contiguous() and k.stride(1) == 1
        kv = torch.empty((n, hd * rep), dtype=torch.uint8, device=k.device)
        vdt = capi.OUT_F16 if value.dtype == torch.float16 else capi.OUT_F32
        capi.check(self.lib.tsattn_kv_product(self.handle, n, n_heads, hd // n_heads, rep, _ptr(k), k.stride(0), vdt, _ptr(value), hd,
                                              float(mult), _ptr(kv), hd * rep, _stream_ptr()))
        return kv

    def matmul_i8(self, a, w, mode=capi.MM_I32, scale=1.0, out=None, workspace=None):
        """MulForward / AddScaled (cpu_infer.cpp:294-316): a uint8 (int8 bytes) [m, k], w uint8 [n, k] (one row per
        output) -> out[m, n]: int32 sums (MM_I32), f32 sums * scale (MM_F32), or out += sums * scale (MM_ADD_SCALED,
        out given, f32)."""
        m, k = a.shape
        n = w.shape[0]
        assert w.shape[1] == k and a.stride(1) == 1 and w.stride(1) == 1
        if mode == capi.MM_I32_PLANES:
            # partial sums [planes, m, n] for a consumer that adds them up (rope_normalize_rows); returns the planes in use
            room = (16 if m <= 128 else 1) * m * n    # K is split only for few rows
            if out is None:
                out = torch.empty(room, dtype=torch.int32, device=a.device)
            assert out.is_contiguous() and out.dtype == torch.int32 and out.numel() >= room
            args = capi.MatmulArgs()
            args.m, args.n, args.k = m, n, k
            args.a, args.a_pitch = _ptr(a), a.stride(0)
            args.w, args.w_pitch = _ptr(w), w.stride(0)
            args.mode, args.scale = mode, 1.0
            args.out, args.out_pitch = _ptr(out), n
            planes = ctypes.c_int(0)
            args.planes_out = ctypes.pointer(planes)
            capi.check(self.lib.tsattn_matmul_i8(self.handle, ctypes.byref(args), _stream_ptr()))
            return out.view(-1)[:planes.value * m * n].view(planes.value, m, n)
        if out is None:
            assert mode != capi.MM_ADD_SCALED
            out = torch.empty((m, n), dtype=torch.int32 if mode == capi.MM_I32 else torch.float32, device=a.device)
        assert out.stride(1) == 1 and out.dtype == (torch.int32 if mode == capi.MM_I32 else torch.float32)
        args = capi.MatmulArgs()
        args.m, args.n, args.k = m, n, k
        args.a, args.a_pitch = _ptr(a), a.stride(0)
        args.w, args.w_pitch = _ptr(w), w.stride(0)
        args.mode, args.scale = mode, float(scale)
        args.out, args.out_pitch = _ptr(out), out.stride(0)
        if workspace is not None:   # a uint8 tensor the caller keeps: room for split-K partial sums when m is small
            args.workspace, args.workspace_bytes = _ptr(workspace), workspace.numel() * workspace.element_size()
        capi.check(self.lib.tsattn_matmul_i8(self.handle, ctypes.byref(args), _stream_ptr()))
        return out

    def embed_rows(self, labels, embed, embed_scale, out=None):
        """The embedding sum of ComputePrediction (cpu_infer.cpp:559-565): labels int32 [n_rows] or [n_rows, L], embed uint8
        (int8 bytes) [n_labels, dim] -> f32 [n_rows, dim]."""
        if labels.dim() == 1:
            labels = labels.view(-1, 1)
        n_rows, per_row = labels.shape
        n_labels, dim = embed.shape
        if out is None:
            out = torch.empty((n_rows, dim), dtype=torch.float32, device=embed.device)
        assert labels.dtype == torch.int32 and labels.is_contiguous() and embed.stride(1) == 1 and out.stride(1) == 1
        capi.check(self.lib.tsattn_embed_rows(self.handle, n_rows, dim, _ptr(labels), per_row, _ptr(embed), embed.stride(0), n_labels,
                                              float(embed_scale), _ptr(out), out.stride(0), _stream_ptr()))
        return out

    def softmax_rows(self, vec, scale, bias=None, want_prob=True, argmax=None):
        """The final SoftMax of ComputePrediction (cpu_infer.cpp:340-355, base 2) and the greedy choice: vec int32 [n_rows, n]
        or [planes, n_rows, n] (parts of a split-K product) -> (prob f32 [n_rows, n] or None, argmax int32 [n_rows])."""
        planes = vec.shape[0] if vec.dim() == 3 else 1
        n_rows, n = vec.shape[-2:]
        assert vec.dtype == torch.int32 and vec.is_contiguous()
        prob = torch.empty((n_rows, n), dtype=torch.float32, device=vec.device) if want_prob else None
        if argmax is None:
            argmax = torch.empty(n_rows, dtype=torch.int32, device=vec.device)
        capi.check(self.lib.tsattn_softmax_rows(self.handle, n_rows, n, _ptr(vec), planes, n_rows * n, n, float(scale), _ptr(bias),
                                                _ptr(prob), n, _ptr(argmax), _stream_ptr()))
        return prob, argmax

    def sample_rows(self, prob, temperature, rnd=None, seed=0, offset=0, choice=None):
        """SampleFromDistr (cpu_infer.cpp:585-599), the Gumbel-max choice: prob f32 [n_rows, n] -> int32 [n_rows].  rnd: the
        caller's uint32 words [n_rows, n], or None = the counter-based generator on (seed, offset)."""
        n_rows, n = prob.shape
        assert prob.dtype == torch.float32 and prob.stride(1) == 1
        if rnd is not None:
            assert rnd.shape == prob.shape and rnd.element_size() == 4 and rnd.stride(1) == 1
        if choice is None:
            choice = torch.empty(n_rows, dtype=torch.int32, device=prob.device)
        capi.check(self.lib.tsattn_sample_rows(self.handle, n_rows, n, _ptr(prob), prob.stride(0), float(temperature), _ptr(rnd),
                                               rnd.stride(0) if rnd is not None else 0, int(seed), int(offset), _ptr(choice),
                                               _stream_ptr()))
        return choice

    def build_spans(self, seq_offset, n_tokens, window, doc_start_flag=None):
        """seq_offset: int32 [n_seqs+1] on the device.  Returns (span_start, span_finish) int32 [n_tokens]."""
        st = torch.empty(n_tokens, dtype=torch.int32, device=self.device)
        fi = torch.empty(n_tokens, dtype=torch.int32, device=self.device)
        capi.check(self.lib.tsattn_build_spans(self.handle, seq_offset.numel() - 1, _ptr(seq_offset), n_tokens,
                                               _ptr(doc_start_flag), int(window), _ptr(st), _ptr(fi), _stream_ptr()))
        return st, fi

    def build_span_tiles(self, span_start, span_finish):
        """Per-128-row summary of a span list for compute_val_lookup(span_tiles=...); build once per batch and mask."""
        n = span_start.numel()
        tiles = torch.empty((self.lib.tsattn_span_tiles_count(n), capi.SPAN_TILE_INTS), dtype=torch.int32, device=self.device)
        capi.check(self.lib.tsattn_build_span_tiles(self.handle, n, _ptr(span_start), _ptr(span_finish), _ptr(tiles),
                                                    _stream_ptr()))
        return tiles

    # ---- prefill --------------------------------------------------------------------------------
    def compute_val_lookup(self, dtype, n_heads, q, k, v, q_scale, k_scale, v_scale, span_start, span_finish,
                           alibi_slope, out=None, out_f16=False, sum_weight_log=None, k_global_scale=None,
                           debug_qk_acc=None, causal_period=0, span_tiles=None, kv_product=None, want_out=True,
                           span_len_hint=0, workspace=None):
        """q,k,v: uint8 [n_tokens, n_heads*d] (row pitch = stride(0)); scales f32 [n_heads, n_tokens] or numbers.
        causal_period: launch-order hint for batches of equal-length sequences under a wide causal window (the
        common sequence length); never changes the result.  span_tiles: what build_span_tiles made of these spans.
        kv_product = (k, kv_out, rep, mult): KVProduct of the f32 result with the tokens' K vectors, written by the same
        launch (k uint8 [n_tokens, H*d], kv_out uint8 [n_tokens, H*rep*d]); with want_out=False the result itself is
        not written and None is returned.
        span_len_hint: typical number of keys per row (the layer's attention width clipped to the sequence length); from
        capi.PREFILL_LONG_SPAN on, with head width 128 and no slope, the call goes through the long-span kernel, which needs a workspace
        (uint8 tensor; by default one that this context keeps and grows on demand)."""
        n_tokens, hd = q.shape
        d = hd // n_heads
        assert want_out or kv_product is not None
        if out is None and want_out:
            out = torch.empty((n_tokens, hd), dtype=torch.float16 if out_f16 else torch.float32, device=q.device)
        a = capi.PrefillArgs()
        a.dtype = dtype
        a.out_dtype = capi.OUT_F16 if (out is not None and out.dtype == torch.float16) else capi.OUT_F32
        a.n_tokens, a.n_heads, a.head_dim = n_tokens, n_heads, d
        a.q, a.k, a.v = _ptr(q), _ptr(k), _ptr(v)
        a.q_pitch, a.k_pitch, a.v_pitch = q.stride(0), k.stride(0), v.stride(0)
        a.q_scale, a.q_scale_const = _scale_arg(q_scale)
        a.k_scale, a.k_scale_const = _scale_arg(k_scale)
        a.v_scale, a.v_scale_const = _scale_arg(v_scale)
        pitches = [s.stride(0) for s in (q_scale, k_scale, v_scale, sum_weight_log) if isinstance(s, torch.Tensor)]
        assert len(set(pitches)) <= 1, "all scale planes must share one pitch"
        a.scale_pitch = pitches[0] if pitches else n_tokens
        a.k_global_scale = _ptr(k_global_scale)
        a.span_start, a.span_finish = _ptr(span_start), _ptr(span_finish)
        if span_start.dim() == 2:      # rows with several spans: [n_parts, n_tokens], part i = every row's i-th span
            assert span_finish.shape == span_start.shape and span_start.stride(1) == 1 and span_finish.stride() == span_start.stride()
            a.n_span_parts, a.span_part_stride = span_start.shape[0], span_start.stride(0)
            assert span_tiles is None or (span_tiles.is_contiguous() and span_tiles.shape[0] == span_start.shape[0])
        a.alibi_slope = float(alibi_slope)
        if out is not None:
            a.out, a.out_pitch = _ptr(out), out.stride(0) * out.element_size()
        a.sum_weight_log = _ptr(sum_weight_log)
        if debug_qk_acc is not None:
            a.debug_qk_acc, a.debug_pitch = _ptr(debug_qk_acc), debug_qk_acc.stride(1)
        if kv_product is not None:
            kv_k, kv_out, kv_rep, kv_mult = kv_product
            assert kv_k.stride(1) == 1 and kv_out.stride(1) == 1
            a.kv_k, a.kv_k_pitch = _ptr(kv_k), kv_k.stride(0)
            a.kv_out, a.kv_out_pitch = _ptr(kv_out), kv_out.stride(0)
            a.kv_rep, a.kv_mult = int(kv_rep), float(kv_mult)
        a.causal_period = int(causal_period)
        a.span_tiles = _ptr(span_tiles)
        a.span_len_hint = int(span_len_hint)
        if span_len_hint >= capi.PREFILL_LONG_SPAN:
            need = int(self.lib.tsattn_prefill_workspace_bytes(n_tokens, n_heads, d))
            if workspace is None and need > 0:
                if self._workspace is None or self._workspace.numel() < need or self._workspace.device != q.device:
                    self._workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
                workspace = self._workspace
            if workspace is not None:
                a.workspace, a.workspace_bytes = _ptr(workspace), workspace.numel() * workspace.element_size()
        capi.check(self.lib.tsattn_prefill(self.handle, ctypes.byref(a), _stream_ptr()))
        return out

    def merge_lookups(self, part_out, part_swl, out=None, out_f16=False, sum_weight_log=None):
        """part_out: f32 [n_parts, n_tokens, H*d], part_swl: f32 [n_parts, H, n_tokens]: prefill results over each row's
        i-th span; returns the attention result over all of a row's spans."""
        n_parts, n_tokens, hd = part_out.shape
        n_heads = part_swl.shape[1]
        if out is None:
            out = torch.empty((n_tokens, hd), dtype=torch.float16 if out_f16 else torch.float32, device=part_out.device)
        a = capi.MergeArgs()
        a.n_parts, a.n_tokens, a.n_heads, a.head_dim = n_parts, n_tokens, n_heads, hd // n_heads
        a.part_out, a.part_out_pitch, a.part_out_stride = _ptr(part_out), part_out.stride(1), part_out.stride(0)
        a.part_swl, a.scale_pitch, a.part_swl_stride = _ptr(part_swl), part_swl.stride(1), part_swl.stride(0)
        a.out_dtype = capi.OUT_F16 if out.dtype == torch.float16 else capi.OUT_F32
        a.out, a.out_pitch = _ptr(out), out.stride(0) * out.element_size()
        if sum_weight_log is not None:
            assert sum_weight_log.stride(0) == a.scale_pitch
            a.sum_weight_log = _ptr(sum_weight_log)
        capi.check(self.lib.tsattn_merge_lookups(self.handle, ctypes.byref(a), _stream_ptr()))
        return out

    def compute_val_lookup_multi(self, dtype, n_heads, q, k, v, q_scale, k_scale, v_scale, span_ptr, spans, alibi_slope,
                                 out_f16=False, sum_weight_log=None, merge=False):
        """Rows with any number of spans, as TAttentionInfo holds them (gpt/att/att.h:24-47): span_ptr int [n_tokens+1],
        spans int [n_spans, 2] (inclusive start, finish), both on the host.  Part i takes every row's i-th span; one
        launch walks all parts (n_span_parts of tsattn_prefill_args), or with merge=True one launch per part and one that
        combines them (tsattn_merge_lookups)."""
        n_tokens = q.shape[0]
        span_ptr = np.asarray(span_ptr, dtype=np.int64)
        spans = np.asarray(spans, dtype=np.int32).reshape(-1, 2)
        counts = span_ptr[1:] - span_ptr[:-1]
        n_parts = max(1, int(counts.max()) if n_tokens else 1)
        st = np.tile(np.arange(n_tokens, dtype=np.int32), (n_parts, 1))
        fi = st - 1                                   # rows that have no i-th span: an empty one
        for i in range(n_parts):
            rows = np.nonzero(counts > i)[0]
            st[i, rows] = spans[span_ptr[rows] + i, 0]
            fi[i, rows] = spans[span_ptr[rows] + i, 1]
        st_d, fi_d = torch.from_numpy(st).to(q.device), torch.from_numpy(fi).to(q.device)
        if not merge:
            return self.compute_val_lookup(dtype, n_heads, q, k, v, q_scale, k_scale, v_scale, st_d, fi_d, alibi_slope,
                                           out_f16=out_f16, sum_weight_log=sum_weight_log)
        part_out = torch.empty((n_parts, n_tokens, q.shape[1]), dtype=torch.float32, device=q.device)
        part_swl = torch.empty((n_parts, n_heads, n_tokens), dtype=torch.float32, device=q.device)
        for i in range(n_parts):
            self.compute_val_lookup(dtype, n_heads, q, k, v, q_scale, k_scale, v_scale, st_d[i], fi_d[i], alibi_slope,
                                    out=part_out[i], sum_weight_log=part_swl[i])
        return self.merge_lookups(part_out, part_swl, out_f16=out_f16, sum_weight_log=sum_weight_log)

    # ---- decode ---------------------------------------------------------------------------------
    def compute_val_lookup_decode(self, cache, q, q_scale, window, alibi_slope, out=None, n_splits=0,
                                  debug_qk_acc=None, max_len=None, append=None, kv_product=None, static_scratch=False):
        """q: uint8 [B, H*d] with q_scale f32 [B, H] (or a number), or bfloat16 [B, H*d] (quantised in the kernel).
        append = (k_new, k_scale_new, v_new, v_scale_new): KVCache.add_vectors fused into the same launches.
        kv_product = (k, kv_out, rep, mult): KVProduct of the result with the token's K vector, written by the same
        launches (k uint8 [B, H*d], kv_out uint8 [B, H*rep*d]).
        static_scratch: go through tsattn_decode_static, the entry point that needs no handle and allocates nothing."""
        B, H, d = cache.n_seqs, cache.n_heads, cache.head_dim
        if out is None:
            out = torch.empty((B, H * d), dtype=torch.float32, device=q.device)
        a = capi.DecodeArgs()
        a.dtype = cache.dtype
        a.q_dtype = capi.Q_BF16 if q.dtype == torch.bfloat16 else capi.Q_8BIT
        a.n_seqs, a.n_heads, a.head_dim = B, H, d
        a.q, a.q_pitch = _ptr(q), q.stride(0) * q.element_size()
        a.q_scale, a.q_scale_const = _scale_arg(q_scale if q_scale is not None else 1.0)
        a.k_cache, a.v_cache = _ptr(cache.k), _ptr(cache.v)
        a.seq_stride, a.head_stride, a.tok_stride = cache.k.stride(0), cache.k.stride(1), cache.k.stride(2)
        a.k_scale, a.k_scale_const = _scale_arg(cache.k_scale)
        a.v_scale, a.v_scale_const = _scale_arg(cache.v_scale)
        if isinstance(cache.k_scale, torch.Tensor):
            a.s_seq_stride, a.s_head_stride = cache.k_scale.stride(0), cache.k_scale.stride(1)
        a.cache_len = _ptr(cache.cache_len)
        a.max_len = cache.max_len if max_len is None else int(max_len)
        a.window = int(window)
        a.alibi_slope = float(alibi_slope)
        a.out = _ptr(out)
        a.n_splits = int(n_splits)
        if debug_qk_acc is not None:
            a.debug_qk_acc, a.debug_pitch = _ptr(debug_qk_acc), debug_qk_acc.stride(1)
        if append is not None:
            k_new, ks_new, v_new, vs_new = append
            a.k_new, a.v_new, a.new_pitch = _ptr(k_new), _ptr(v_new), k_new.stride(0)
            a.k_scale_new, a.v_scale_new = _ptr(ks_new), _ptr(vs_new)
        if kv_product is not None:
            kk, kv_out, rep, mult = kv_product
            a.kv_k, a.kv_k_pitch, a.kv_out, a.kv_out_pitch = _ptr(kk), kk.stride(0), _ptr(kv_out), kv_out.stride(0)
            a.kv_rep, a.kv_mult = int(rep), float(mult)
        if static_scratch:
            capi.check(self.lib.tsattn_decode_static(ctypes.byref(a), _stream_ptr()))
        else:
            capi.check(self.lib.tsattn_decode(self.handle, ctypes.byref(a), _stream_ptr()))
        return out


VEC_SCALE = 1.0 / 24      # gpt/train/cpu_infer.cpp:16
STATE_NORM_TILE = 128     # gpt/model_params/model_dim.h:22
COMBINER_REP = 4          # gpt/model_params/model_dim.h:12


def add_lookup_product(ctx, layer, cache, t, rope, state, workspace=None, scratch=None, pending=None, defer=False):
    """One layer of the int8 inference path for one new token per sequence: AddLookupProduct,
    gpt/train/cpu_infer.cpp:465-527, as a chain of 10-11 library calls (the C++ form is NTsAttn::TLayerComputer).
    layer: dict with uint8 (int8 bytes) matrices proj [4*H*d, dim] (the QK, QV, K and V matrices one after the other),
    combiner [dim, 4*H*d], expand [H*d, dim], contract [dim, H*d], floats qv_scale, combiner_scale, contract_scale, and
    width, slope.  cache: KVCache whose value scales are VEC_SCALE; t: int32 [B] positions; rope: table of
    fill_rope_table; state: f32 [B, dim], updated in place.  scratch: dict for buffers kept between calls.
    Returns the attention output [B, H*d].
    defer=True leaves the layer's last state update (contract's AddScaled) undone and returns (attention output,
    pending): the next layer's first normalisation does it when given `pending` (one launch less per layer), and
    flush_state does it after the last layer."""
    B, dim = state.shape
    H, d = cache.n_heads, cache.head_dim
    qsum = H * d
    groups = dim // STATE_NORM_TILE
    f32 = np.float32
    sc = scratch if scratch is not None else {}
    if "planes" not in sc:
        sc["planes"] = torch.empty((16, B, max(4 * qsum, dim, layer["expand"].shape[0])), dtype=torch.int32, device=state.device)
        sc["v_scale"] = torch.full((B, H), VEC_SCALE, dtype=torch.float32, device=state.device)
    planes_buf, v_scale = sc["planes"], sc["v_scale"]
    if pending is not None:   # the previous layer's contract product, still in parts: state += sum * scale, then normalise
        norm, _ = ctx.rope_normalize_rows(pending[0], groups, capi.I8, resid=state, resid_scale=pending[1])
    else:
        norm, _ = ctx.rope_normalize_rows(state, groups, capi.I8)
    # the four projections as one product; RoPE on the qk and qv heads, per-head normalisation of all four in one call
    proj = ctx.matmul_i8(norm, layer["proj"], mode=capi.MM_I32_PLANES, out=planes_buf)
    key_mult = float(f32(layer["qv_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(dim))))
    q4, qv_scale = ctx.rope_normalize_rows(proj, 4 * H, capi.I8, pos=t, rope=rope, scale_mult=key_mult, row_major_scale=True,
                                           rope_heads=2 * H, scale_heads=(H, H))
    qk, qv, k, v = q4[:, :qsum], q4[:, qsum:2 * qsum], q4[:, 2 * qsum:3 * qsum], q4[:, 3 * qsum:]
    if "kv" not in sc:
        sc["kv"] = torch.empty((B, qsum * COMBINER_REP), dtype=torch.uint8, device=state.device)
        sc["val"] = torch.empty((B, qsum), dtype=torch.float32, device=state.device)
    kv, val = sc["kv"], sc["val"]
    fused_kv = (k, kv, COMBINER_REP, 1.0)   # KVProduct written by the attention launches themselves
    if layer["width"] == 0:   # the token attends to the row being written: append first
        cache.add_vectors(qv, qv_scale, v, v_scale)
        ctx.compute_val_lookup_decode(cache, qk, VEC_SCALE, 0, layer["slope"], out=val, kv_product=fused_kv)
    else:
        ctx.compute_val_lookup_decode(cache, qk, VEC_SCALE, layer["width"], layer["slope"], out=val, append=(qv, qv_scale, v, v_scale),
                                      kv_product=fused_kv)
    # combiner; its AddScaled is done by the normalisation that follows
    delta = ctx.matmul_i8(kv, layer["combiner"], mode=capi.MM_I32_PLANES, out=planes_buf)
    norm, _ = ctx.rope_normalize_rows(delta, groups, capi.I8, resid=state,
                                      resid_scale=float(f32(layer["combiner_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(qsum * COMBINER_REP)))))
    relu_src = ctx.matmul_i8(norm, layer["expand"], mode=capi.MM_I32_PLANES, out=planes_buf)
    relu, _ = ctx.rope_normalize_rows(relu_src, H, capi.I8, relu=True)
    relu_dim = relu_src.shape[-1]
    contract_scale = float(f32(layer["contract_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(relu_dim))))
    if defer:
        parts = ctx.matmul_i8(relu, layer["contract"], mode=capi.MM_I32_PLANES, out=planes_buf)
        return val, (parts, contract_scale)
    ctx.matmul_i8(relu, layer["contract"], mode=capi.MM_ADD_SCALED, out=state, workspace=workspace, scale=contract_scale)
    return val


def flush_state(ctx, pending, state):
    """The state update a deferred add_lookup_product left undone; returns NormalizeState of the updated state (what
    ComputePrediction multiplies with the final layer)."""
    norm, _ = ctx.rope_normalize_rows(pending[0], state.shape[1] // STATE_NORM_TILE, capi.I8, resid=state, resid_scale=pending[1])
    return norm


def add_lookup_product_prompt(ctx, layer, cache, seq_offset, pos, rope, state, span_start, span_finish, span_tiles=None,
                              causal_period=0, norm=None, want_norm=False, want_val=True):
    """The same layer for a whole batch of prompt tokens at once (sequences concatenated, seq_offset int32 [B+1], pos
    int32 [n_tokens] = each token's position in its sequence): every token's attention over the earlier tokens of its
    sequence is one tsattn_prefill launch, and the tokens' key and value rows go into the cache in one
    tsattn_cache_fill.  Token by token through add_lookup_product gives the same cache and the same states (a token's
    layer input does not depend on other tokens' outputs of the same layer).  state: f32 [n_tokens, dim], updated in
    place; the spans are those of the layer's width (build_spans).  Returns the attention output (None with
    want_val=False: KVProduct is the attention kernel's last step and nothing else reads the output).
    norm: NormalizeState(state) where the caller has it (the previous layer's second result); want_norm=True returns
    (attention output, NormalizeState(new state)), which the layer's last product then makes as its epilogue."""
    n, dim = state.shape
    H, d = cache.n_heads, cache.head_dim
    qsum = H * d
    groups = dim // STATE_NORM_TILE
    f32 = np.float32
    if norm is None:
        norm, _ = ctx.rope_normalize_rows(state, groups, capi.I8)
    # every product with its normalisation as epilogue (large products never write their int32 sums); one scratch
    # buffer for whichever falls back to two launches
    key_mult = float(f32(layer["qv_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(dim))))
    room = torch.empty((16 if n <= 128 else 1) * n * max(4 * qsum, dim, layer["expand"].shape[0]), dtype=torch.int32, device=state.device)
    q4, qv_scale = ctx.matmul_normalize(norm, layer["proj"], 4 * H, capi.I8, room, pos=pos, rope=rope, scale_mult=key_mult,
                                        rope_heads=2 * H, scale_heads=(H, H))      # scales as [head][token] planes
    qk, qv, k, v = q4[:, :qsum], q4[:, qsum:2 * qsum], q4[:, 2 * qsum:3 * qsum], q4[:, 3 * qsum:]
    # attention with KVProduct as its last step: the result itself is written only for a caller who wants it
    kv = torch.empty((n, qsum * COMBINER_REP), dtype=torch.uint8, device=state.device)
    val = ctx.compute_val_lookup(capi.I8, H, qk, qv, v, VEC_SCALE, qv_scale, VEC_SCALE, span_start, span_finish, layer["slope"],
                                 span_tiles=span_tiles, causal_period=causal_period, kv_product=(k, kv, COMBINER_REP, 1.0),
                                 want_out=want_val)
    cache.fill_from_prefill(seq_offset, qv, qv_scale, v)       # value scales: the cache's constant VEC_SCALE
    norm, _ = ctx.matmul_normalize(kv, layer["combiner"], groups, capi.I8, room, resid=state,
                                   resid_scale=float(f32(layer["combiner_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(qsum * COMBINER_REP)))))
    del kv
    relu, _ = ctx.matmul_normalize(norm, layer["expand"], H, capi.I8, room, relu=True)
    relu_dim = relu.shape[-1]
    contract_scale = float(f32(layer["contract_scale"]) * f32(VEC_SCALE) * f32(np.sqrt(f32(1.0) / f32(relu_dim))))
    if want_norm:   # state += product * scale, and the updated state normalised for whoever comes next
        norm_next, _ = ctx.matmul_normalize(relu, layer["contract"], groups, capi.I8, room, resid=state, resid_scale=contract_scale)
        return val, norm_next
    del room
    ctx.matmul_i8(relu, layer["contract"], mode=capi.MM_ADD_SCALED, out=state, scale=contract_scale)
    return val


class KVCache:
    """Planar KV cache [n_seqs][n_heads][max_len][d] 8-bit with f32 row scales [n_seqs][n_heads][max_len];
    the device-resident counterpart of TAttentionVecHistory (gpt/train/cpu_infer.cpp:397-410)."""

    def __init__(self, ctx, dtype, n_seqs, n_heads, max_len, head_dim, const_scales=None):
        dev = ctx.device
        self.ctx, self.dtype = ctx, dtype
        self.n_seqs, self.n_heads, self.max_len, self.head_dim = n_seqs, n_heads, max_len, head_dim
        self.k = torch.zeros((n_seqs, n_heads, max_len, head_dim), dtype=torch.uint8, device=dev)
        self.v = torch.zeros_like(self.k)
        if const_scales is None:
            self.k_scale = torch.zeros((n_seqs, n_heads, max_len), dtype=torch.float32, device=dev)
            self.v_scale = torch.zeros_like(self.k_scale)
        else:
            self.k_scale, self.v_scale = const_scales
        self.cache_len = torch.zeros(n_seqs, dtype=torch.int32, device=dev)

    def add_vectors(self, k_new, k_scale_new, v_new, v_scale_new=None):
        """k_new, v_new: uint8 [n_seqs, n_heads*d]; scales f32 [n_seqs, n_heads] (None with constant scales)."""
        a = capi.AppendArgs()
        a.n_seqs, a.n_heads, a.head_dim = self.n_seqs, self.n_heads, self.head_dim
        a.k_new, a.v_new, a.new_pitch = _ptr(k_new), _ptr(v_new), k_new.stride(0)
        a.k_scale_new, a.v_scale_new = _ptr(k_scale_new), _ptr(v_scale_new)
        a.k_cache, a.v_cache = _ptr(self.k), _ptr(self.v)
        a.seq_stride, a.head_stride, a.tok_stride = self.k.stride(0), self.k.stride(1), self.k.stride(2)
        if isinstance(self.k_scale, torch.Tensor):
            a.k_scale, a.v_scale = _ptr(self.k_scale), _ptr(self.v_scale)
            a.s_seq_stride, a.s_head_stride = self.k_scale.stride(0), self.k_scale.stride(1)
        a.cache_len, a.max_len = _ptr(self.cache_len), self.max_len
        capi.check(self.ctx.lib.tsattn_cache_append(self.ctx.handle, ctypes.byref(a), _stream_ptr()))

    def fill_from_prefill(self, seq_offset, k, k_scale, v, v_scale=None):
        """Append a prefill batch: k, v uint8 [n_tokens, n_heads*d]; scales f32 [n_heads, n_tokens] planes (None
        with constant scales); seq_offset int32 [n_seqs+1] on the device.  Equals add_vectors once per token."""
        a = capi.FillArgs()
        a.n_seqs, a.n_heads, a.head_dim = self.n_seqs, self.n_heads, self.head_dim
        a.n_tokens = k.shape[0]
        a.seq_offset = _ptr(seq_offset)
        a.k, a.v, a.pitch = _ptr(k), _ptr(v), k.stride(0)
        assert v.stride(0) == k.stride(0)
        a.k_scale, a.v_scale = _ptr(k_scale), _ptr(v_scale)
        pitches = [s.stride(0) for s in (k_scale, v_scale) if s is not None]
        assert len(set(pitches)) <= 1
        a.scale_pitch = pitches[0] if pitches else a.n_tokens
        a.k_cache, a.v_cache = _ptr(self.k), _ptr(self.v)
        a.seq_stride, a.head_stride, a.tok_stride = self.k.stride(0), self.k.stride(1), self.k.stride(2)
        if isinstance(self.k_scale, torch.Tensor):
            a.k_scale_cache, a.v_scale_cache = _ptr(self.k_scale), _ptr(self.v_scale)
            a.s_seq_stride, a.s_head_stride = self.k_scale.stride(0), self.k_scale.stride(1)
        a.cache_len, a.max_len = _ptr(self.cache_len), self.max_len
        capi.check(self.ctx.lib.tsattn_cache_fill(self.ctx.handle, ctypes.byref(a), _stream_ptr()))
