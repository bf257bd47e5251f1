"""GPU: tsattn_decode_static, the decode entry point that allocates nothing (its split partials and arrival counters are
an array in the library's device image), against tsattn_decode with a handle: same kernels, so the outputs, the caches
and the lengths must be identical.  Two calls in a row on the shared array, the second with a smaller input; with several
splits (partials and merge), one split, and the fused append (arrival counters)."""
import numpy as np
import pytest
import torch

from tscale_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=64, max_heads=16, max_head_dim=128, max_splits=32)
    yield c
    c.close()


def filled_cache(ctx, seed, B, H, L, d, lens):
    from tscale_amd import KVCache
    g = torch.Generator(device="cuda").manual_seed(seed)
    c = KVCache(ctx, capi.I8, B, H, L, d)
    c.k.copy_(torch.randint(-127, 128, (B, H, L, d), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8))
    c.v.copy_(torch.randint(-127, 128, (B, H, L, d), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8))
    c.k_scale.copy_((torch.rand((B, H, L), device="cuda", generator=g) + 0.5) * 2e-3)
    c.v_scale.copy_((torch.rand((B, H, L), device="cuda", generator=g) + 0.5) / 24)
    c.cache_len.copy_(torch.tensor(lens, dtype=torch.int32))
    return c


def clone_cache(ctx, c):
    from tscale_amd import KVCache
    n = KVCache(ctx, c.dtype, c.n_seqs, c.n_heads, c.max_len, c.head_dim)
    for a in ("k", "v", "k_scale", "v_scale", "cache_len"):
        getattr(n, a).copy_(getattr(c, a))
    return n


@pytest.mark.parametrize("splits", [0, 1, 4])
def test_two_calls_in_a_row_equal_the_handle_path(ctx, splits):
    for call, (B, H, L, d) in enumerate(((16, 16, 1500, 128), (5, 3, 300, 64))):   # the second, smaller call reuses the array
        rng = np.random.default_rng(40 + call)
        lens = [int(x) for x in rng.integers(1, L + 1, B)]
        lens[0] = L
        cache = filled_cache(ctx, 7 + call, B, H, L, d, lens)
        g = torch.Generator(device="cuda").manual_seed(100 + call)
        q = torch.randn((B, H * d), device="cuda", generator=g).to(torch.bfloat16)
        want = ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.25, n_splits=splits)
        got = ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.25, n_splits=splits, static_scratch=True)
        assert torch.equal(got, want), (call, splits, (got - want).abs().max().item())
        assert bool(torch.isfinite(got).all()) and float(got.abs().max()) > 0


def test_fused_append_through_the_static_entry_point(ctx):
    for call, (B, H, L, d) in enumerate(((12, 8, 700, 128), (3, 2, 90, 128))):
        rng = np.random.default_rng(60 + call)
        lens = [int(x) for x in rng.integers(0, L, B)]
        a = filled_cache(ctx, 17 + call, B, H, L, d, lens)
        b = clone_cache(ctx, a)
        g = torch.Generator(device="cuda").manual_seed(200 + call)
        x = torch.randn((3, B, H * d), device="cuda", generator=g)
        q, qs = ctx.quantize_rows(x[0], H, capi.I8)
        kn, kns = ctx.quantize_rows(x[1], H, capi.I8)
        vn, vns = ctx.quantize_rows(x[2], H, capi.I8)
        qs, kns, vns = (s.t().contiguous() for s in (qs, kns, vns))
        for window in (64, 10 ** 6):   # one split (counters), then the library's choice
            want = ctx.compute_val_lookup_decode(a, q, qs, window, 0.5, append=(kn, kns, vn, vns))
            got = ctx.compute_val_lookup_decode(b, q, qs, window, 0.5, append=(kn, kns, vn, vns), static_scratch=True)
            assert torch.equal(got, want), (call, window)
            for name in ("k", "v", "k_scale", "v_scale", "cache_len"):
                assert torch.equal(getattr(a, name), getattr(b, name)), (call, window, name)


def test_no_device_memory_is_taken(ctx):
    """Free device memory, as the driver reports it, is the same before and after static calls -- the first one of the
    process on this device included when this file runs alone (the array is part of the library's device image)."""
    B, H, L, d = 8, 4, 600, 128
    cache = filled_cache(ctx, 31, B, H, L, d, [L] * B)
    q = torch.randn((B, H * d), device="cuda").to(torch.bfloat16)
    out = torch.empty((B, H * d), dtype=torch.float32, device="cuda")
    want = ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.0, n_splits=4)   # (the kernels' code is loaded by now)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.0, n_splits=4, out=out, static_scratch=True)
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0, (free0, free1)
    assert torch.equal(out, want)


def test_static_fused_append_in_a_graph(ctx):
    """The static entry point under stream capture, without help from a handle's buffers: a fused-append decode with one
    split (window 64: the arrival counters in the array are used, and cleared by the fill kernel in front of the launch),
    replayed three times with eager work between the replays, every replay against eager calls on a copy of the cache."""
    B, H, L, d = 6, 4, 300, 128
    rng = np.random.default_rng(77)
    lens = [int(x) for x in rng.integers(70, L - 8, B)]
    a = filled_cache(ctx, 23, B, H, L, d, lens)
    b = clone_cache(ctx, a)
    g0 = torch.Generator(device="cuda").manual_seed(300)
    x = torch.randn((3, B, H * d), device="cuda", generator=g0)
    q, qs = ctx.quantize_rows(x[0], H, capi.I8)
    kn, kns = ctx.quantize_rows(x[1], H, capi.I8)
    vn, vns = ctx.quantize_rows(x[2], H, capi.I8)
    qs, kns, vns = (s.t().contiguous() for s in (qs, kns, vns))
    out = torch.zeros((B, H * d), dtype=torch.float32, device="cuda")
    step = lambda: ctx.compute_val_lookup_decode(b, q, qs, 64, 0.5, out=out, append=(kn, kns, vn, vns), static_scratch=True)
    # warm up on a side stream (as torch asks), put the cache back, record
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for name in ("k", "v", "k_scale", "v_scale", "cache_len"):
        getattr(b, name).copy_(getattr(a, name))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    torch.cuda.synchronize()
    for name in ("k", "v", "k_scale", "v_scale", "cache_len"):   # (capture runs nothing, but the cache is put back all the same)
        getattr(b, name).copy_(getattr(a, name))
    for replay in range(3):
        want = ctx.compute_val_lookup_decode(a, q, qs, 64, 0.5, append=(kn, kns, vn, vns))   # eager, handle path
        float((torch.randn(1 << 16, device="cuda") * 2 + 1).sum())                           # eager work of the program's own
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
        for name in ("k", "v", "k_scale", "v_scale", "cache_len"):
            assert torch.equal(getattr(a, name), getattr(b, name)), (replay, name)


def test_limits_are_refused_with_a_clear_error(ctx):
    from tscale_amd import KVCache
    B, H, L, d = 40, 16, 64, 64
    cache = KVCache(ctx, capi.I8, B, H, L, d)
    cache.cache_len.fill_(L)
    q = torch.zeros((B, H * d), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds the scratch"):
        ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.0, n_splits=32, static_scratch=True)   # 40 * 16 * 32 parts
