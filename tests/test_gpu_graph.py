"""GPU: the calls can be recorded into a HIP graph and replayed (the reference runs its kernels as nodes of a pre-built
graph, lib/cuda/cuda_graph.cuh:92-125, 259-272): no call synchronises, allocates or reads device data on the host.  Each
graph is replayed three times with eager work of the program's own and synchronisations between the replays, and every
replay is compared with the same calls made eagerly on a copy of the state."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tscale_amd import KVCache, capi
from tscale_amd.attention import VEC_SCALE, add_lookup_product

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=16, max_heads=8, max_head_dim=128, max_splits=32)
    yield c
    c.close()


def capture(fn):
    """Warm up on a side stream (as torch asks), then record fn into a graph."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    torch.cuda.synchronize()
    return g


def counters(ctx, n):
    dst = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    capi.check(ctx.lib.tsattn_debug_read_counters(ctx.handle, ctypes.c_void_p(dst.data_ptr()), n, None))
    torch.cuda.synchronize()
    return dst.cpu().tolist()


def clone_cache(ctx, c):
    n = KVCache(ctx, c.dtype, c.n_seqs, c.n_heads, c.max_len, c.head_dim)
    for a in ("k", "v", "k_scale", "v_scale", "cache_len"):
        getattr(n, a).copy_(getattr(c, a))
    return n


def eager_noise():
    x = torch.randn(1 << 16, device="cuda")
    return float((x * 2 + 1).sum())


def test_long_span_prefill_replays(ctx):
    """The long-span kernel and the kernel that writes its copy of V into the caller's workspace, as two nodes of a graph."""
    dtype, H, d, n = capi.E4M3, 4, 128, 900
    g0 = torch.Generator(device="cuda").manual_seed(6)
    q, qs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    k, ks = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    v, vs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    off = torch.tensor([0, n], dtype=torch.int32, device="cuda")
    st, fi = ctx.build_spans(off, n, 10 ** 6)
    hint = capi.PREFILL_LONG_SPAN
    want = ctx.compute_val_lookup(dtype, H, q, k, v, qs, ks, vs, st, fi, 0.0, span_len_hint=hint).clone()   # (allocates the workspace)
    out = torch.zeros_like(want)
    graph = capture(lambda: ctx.compute_val_lookup(dtype, H, q, k, v, qs, ks, vs, st, fi, 0.0, out=out, span_len_hint=hint))
    for _ in range(3):
        out.zero_()
        ctx._workspace.fill_(0xFF)   # the copy of V is made again by every replay (0xFF..: NaN halves)
        eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


@pytest.mark.parametrize("dtype,window,slope", [(capi.E4M3, 10 ** 6, 0.0), (capi.I8, 64, 0.5)])
def test_prefill_replays(ctx, dtype, window, slope):
    H, d, lens = 4, 128, [300, 77, 513]
    n = sum(lens)
    g0 = torch.Generator(device="cuda").manual_seed(5)
    q, qs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    k, ks = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    v, vs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    off = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device="cuda")
    st, fi = ctx.build_spans(off, n, window)
    want = ctx.compute_val_lookup(dtype, H, q, k, v, qs, ks, vs, st, fi, slope).clone()
    out = torch.zeros_like(want)
    graph = capture(lambda: ctx.compute_val_lookup(dtype, H, q, k, v, qs, ks, vs, st, fi, slope, out=out))
    for _ in range(3):
        out.zero_()
        eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_several_spans_per_row_replay(ctx):
    """Two prefill launches over the rows' first and second spans and the launch that combines them, as one graph."""
    dtype, H, d, n = capi.I8, 2, 128, 400
    g0 = torch.Generator(device="cuda").manual_seed(9)
    q, qs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    k, ks = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    v, vs = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g0), H, dtype)
    t = torch.arange(n, dtype=torch.int32, device="cuda")
    spans = [(torch.clamp(t - 40, min=0), t - 1), (torch.zeros_like(t), torch.clamp(t - 300, min=-1))]   # a window and a far prefix
    parts = torch.zeros((2, n, H * d), dtype=torch.float32, device="cuda")
    swl = torch.zeros((2, H, n), dtype=torch.float32, device="cuda")
    out = torch.zeros((n, H * d), dtype=torch.float32, device="cuda")
    def run():
        for i, (st, fi) in enumerate(spans):
            ctx.compute_val_lookup(dtype, H, q, k, v, qs, ks, vs, st.contiguous(), fi.contiguous(), 0.25, out=parts[i], sum_weight_log=swl[i])
        ctx.merge_lookups(parts, swl, out=out)
    run()
    torch.cuda.synchronize()
    want = out.clone()
    assert want.abs().max() > 0
    graph = capture(run)
    for _ in range(3):
        out.zero_(); parts.zero_(); swl.zero_()
        eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


@pytest.mark.parametrize("window,splits", [(64, 1), (10 ** 6, 0), (10 ** 6, 5)])
def test_fused_append_and_decode_replays(ctx, window, splits):
    """Every replay appends one more row per sequence and attends over the longer cache; the arrival counters of the
    single-split form are back at zero after each."""
    B, H, L, d = 6, 8, 900, 128
    g0 = torch.Generator(device="cuda").manual_seed(9)
    a = KVCache(ctx, capi.I8, B, H, L, d)
    a.k.copy_(torch.randint(-127, 128, (B, H, L, d), dtype=torch.int8, device="cuda", generator=g0).view(torch.uint8))
    a.v.copy_(torch.randint(-127, 128, (B, H, L, d), dtype=torch.int8, device="cuda", generator=g0).view(torch.uint8))
    a.k_scale.copy_((torch.rand((B, H, L), device="cuda", generator=g0) + 0.5) * 2e-3)
    a.v_scale.copy_((torch.rand((B, H, L), device="cuda", generator=g0) + 0.5) / 24)
    a.cache_len.copy_(torch.tensor([0, 1, 63, 500, 896, 899], dtype=torch.int32))
    b = clone_cache(ctx, a)        # the graph's cache
    fresh = clone_cache(ctx, a)
    x = torch.randn((3, B, H * d), device="cuda", generator=g0)
    q, qs = ctx.quantize_rows(x[0], H, capi.I8)
    kn, kns = ctx.quantize_rows(x[1], H, capi.I8)
    vn, vns = ctx.quantize_rows(x[2], H, capi.I8)
    qs, kns, vns = (s.t().contiguous() for s in (qs, kns, vns))
    out = torch.zeros((B, H * d), device="cuda")
    call = lambda cache, o: ctx.compute_val_lookup_decode(cache, q, qs, window, 0.25, out=o, n_splits=splits, append=(kn, kns, vn, vns))
    graph = capture(lambda: call(b, out))
    for name in ("k", "v", "k_scale", "v_scale", "cache_len"):     # the warm-up and the capture must not count
        getattr(b, name).copy_(getattr(fresh, name))
    assert counters(ctx, B) == [0] * B
    for rep in range(3):
        want = call(a, torch.zeros_like(out)).clone()
        eager_noise()
        out.fill_(-7.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        for name in ("k", "v", "k_scale", "v_scale", "cache_len"):
            assert torch.equal(getattr(a, name), getattr(b, name)), (rep, name)
        assert counters(ctx, B) == [0] * B, rep
    assert b.cache_len.cpu().tolist() == [3, 4, 66, 503, 899, 900]   # the last one filled up after one row


def test_layer_step_replays(ctx):
    """One token through one int8 layer (AddLookupProduct, gpt/train/cpu_infer.cpp:465-527) as a graph: the chain of
    library calls -- normalisations, products, fused append + decode + KVProduct, residual updates."""
    B, H, d, dim, max_len = 4, 2, 128, 256, 16
    qsum = H * d
    rng = np.random.default_rng(31)
    mat = lambda r, k: np.clip(np.rint(rng.standard_normal((r, k)) * 32), -127, 127).astype(np.int8)
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()
    layer = {"proj": dev(np.concatenate([mat(qsum, dim) for _ in range(4)]).view(np.uint8)), "combiner": dev(mat(dim, qsum * 4).view(np.uint8)),
             "expand": dev(mat(qsum, dim).view(np.uint8)), "contract": dev(mat(dim, qsum).view(np.uint8)),
             "qv_scale": 0.031, "combiner_scale": 0.027, "contract_scale": 0.035, "width": 1000, "slope": 0.0}
    a = KVCache(ctx, capi.I8, B, H, max_len, d)
    a.k.copy_(dev(rng.integers(-127, 128, (B, H, max_len, d)).astype(np.int8).view(np.uint8)))
    a.v.copy_(dev(rng.integers(-127, 128, (B, H, max_len, d)).astype(np.int8).view(np.uint8)))
    a.k_scale.copy_(dev(((rng.random((B, H, max_len)) + 0.5) * 1e-3).astype(np.float32)))
    a.v_scale.fill_(VEC_SCALE)
    a.cache_len.copy_(dev(np.array([0, 2, 7, 9], dtype=np.int32)))
    b, fresh = clone_cache(ctx, a), clone_cache(ctx, a)
    rope = dev(orc.fill_rope(d, 64))
    t = dev(np.array([3, 5, 10, 12], dtype=np.int32))
    state0 = dev(rng.standard_normal((B, dim)).astype(np.float32) * 2)
    sa, sb = state0.clone(), state0.clone()
    room_a = torch.empty(16 * 4 * B * dim * 8, dtype=torch.uint8, device="cuda")
    room_b = torch.empty_like(room_a)
    keep_a, keep_b = {}, {}
    graph = capture(lambda: add_lookup_product(ctx, layer, b, t, rope, sb, workspace=room_b, scratch=keep_b))
    sb.copy_(state0)
    for name in ("k", "v", "k_scale", "v_scale", "cache_len"):
        getattr(b, name).copy_(getattr(fresh, name))
    for rep in range(3):
        add_lookup_product(ctx, layer, a, t, rope, sa, workspace=room_a, scratch=keep_a)
        eager_noise()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(sa, sb), rep
        for name in ("k", "v", "k_scale", "cache_len"):
            assert torch.equal(getattr(a, name), getattr(b, name)), (rep, name)
        assert bool(torch.isfinite(sb).all())
    assert b.cache_len.cpu().tolist() == [3, 5, 10, 12]
