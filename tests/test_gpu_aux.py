"""GPU: the quantiser, span builder and cache append of libtsattn.so against the oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tscale_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=64, max_heads=16, max_head_dim=128)
    yield c
    c.close()


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("d", [64, 128])
def test_quantize_rows_bit_exact(ctx, dtype, d):
    H, n = 3, 257
    x = np.random.default_rng(40 + d).standard_normal((n, H * d)).astype(np.float32)
    x[5, d:2 * d] = 0
    x[6] *= 1e-20
    x[7] *= 1e20
    want_q, want_s = orc.quantize_rows(dtype, x, H)
    q, s = ctx.quantize_rows(torch.from_numpy(x).cuda(), H, dtype)
    assert np.array_equal(s.cpu().numpy(), want_s)
    got = q.cpu().numpy()
    if dtype == capi.E4M3:  # -0 and +0 are the same value
        got = np.where((got & 0x7F) == 0, 0, got)
        want_q = np.where((want_q & 0x7F) == 0, 0, want_q)
    assert np.array_equal(got, want_q)


def test_quantize_rows_bf16_source(ctx):
    H, d, n = 2, 128, 33
    x = torch.randn((n, H * d), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    want_q, want_s = orc.quantize_rows(orc.I8, bits, H)
    q, s = ctx.quantize_rows(x.cuda(), H, capi.I8)
    assert np.array_equal(q.cpu().numpy(), want_q) and np.array_equal(s.cpu().numpy(), want_s)


@pytest.mark.parametrize("window", [0, 1, 64, 5000])
def test_build_spans_matches_oracle(ctx, window):
    seq_lens = [1, 300, 2, 1024, 77]
    n = sum(seq_lens)
    off = np.zeros(len(seq_lens) + 1, np.int32)
    off[1:] = np.cumsum(seq_lens)
    for flags in (None, (np.random.default_rng(1).random(n) < 0.02).astype(np.uint8)):
        st, fi = orc.make_spans(seq_lens, window, flags)
        gst, gfi = ctx.build_spans(torch.from_numpy(off).cuda(), n, window,
                                   None if flags is None else torch.from_numpy(flags).cuda())
        assert np.array_equal(gst.cpu().numpy(), st) and np.array_equal(gfi.cpu().numpy(), fi)


def test_cache_append(ctx):
    from tscale_amd import KVCache
    B, H, L, d = 3, 2, 5, 64
    cache = KVCache(ctx, capi.I8, B, H, L, d)
    cache.cache_len.copy_(torch.tensor([0, 4, 5], dtype=torch.int32))  # last one is full
    g = torch.Generator().manual_seed(0)
    k = torch.randint(0, 256, (B, H * d), dtype=torch.uint8, generator=g).cuda()
    v = torch.randint(0, 256, (B, H * d), dtype=torch.uint8, generator=g).cuda()
    ks = torch.rand((B, H), generator=g).cuda()
    vs = torch.rand((B, H), generator=g).cuda()
    cache.add_vectors(k, ks, v, vs)
    torch.cuda.synchronize()
    assert cache.cache_len.tolist() == [1, 5, 5]
    kc = cache.k.cpu()
    assert torch.equal(kc[0, :, 0].reshape(-1), k[0].cpu()) and torch.equal(kc[1, :, 4].reshape(-1), k[1].cpu())
    assert torch.equal(cache.v.cpu()[1, :, 4].reshape(-1), v[1].cpu())
    assert torch.equal(cache.k_scale.cpu()[0, :, 0], ks[0].cpu()) and torch.equal(cache.v_scale.cpu()[1, :, 4], vs[1].cpu())
    assert not kc[2].any() and not kc[0, :, 1:].any()


def test_error_paths(ctx):
    from tscale_amd.capi import TsattnError
    q = torch.zeros((4, 96), dtype=torch.uint8, device="cuda")
    sp = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(TsattnError) as e:
        ctx.compute_val_lookup(capi.I8, 1, q, q, q, 1.0, 1.0, 1.0, sp, sp, 0.0)  # head_dim 96
    assert e.value.code == 2 and "head_dim" in str(e.value)
    with pytest.raises(TsattnError) as e:
        ctx.compute_val_lookup(7, 1, q[:, :64], q[:, :64], q[:, :64], 1.0, 1.0, 1.0, sp, sp, 0.0)
    assert e.value.code in (1, 2)


@pytest.mark.parametrize("d", [64, 128])
def test_cache_fill_equals_token_by_token_append(ctx, d):
    """The bulk append of a prefill batch writes what AddVectors would write one token at a time
    (cpu_infer.cpp:403-408): ragged sequences, an empty one, caches that already hold rows, one that overflows."""
    from tscale_amd import KVCache
    B, H, L = 5, 3, 40
    lens = [17, 0, 33, 1, 25]
    start = [0, 3, 5, 39, 30]     # the last sequence would reach 55 rows: rows beyond 40 are dropped
    off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    n = int(off[-1])
    g = torch.Generator().manual_seed(d)
    k = torch.randint(0, 256, (n, H * d), dtype=torch.uint8, generator=g).cuda()
    v = torch.randint(0, 256, (n, H * d), dtype=torch.uint8, generator=g).cuda()
    ks = torch.rand((H, n), generator=g).cuda()
    vs = torch.rand((H, n), generator=g).cuda()

    bulk = KVCache(ctx, capi.I8, B, H, L, d)
    bulk.cache_len.copy_(torch.tensor(start, dtype=torch.int32))
    bulk.fill_from_prefill(torch.from_numpy(off).cuda(), k, ks, v, vs)

    single = KVCache(ctx, capi.I8, B, H, L, d)
    single.cache_len.copy_(torch.tensor(start, dtype=torch.int32))
    # token-by-token: sequences that have run out of tokens are parked on a full cache_len (= no-op)
    for t in range(max(lens)):
        rows = [int(off[b]) + min(t, max(lens[b] - 1, 0)) for b in range(B)]
        kk = k[rows].contiguous(); vv = v[rows].contiguous()
        kss = ks[:, rows].t().contiguous(); vss = vs[:, rows].t().contiguous()
        active = torch.tensor([t < lens[b] for b in range(B)]).cuda()
        saved = single.cache_len.clone()
        single.cache_len.copy_(torch.where(active, saved, torch.full_like(saved, L)))
        single.add_vectors(kk, kss, vv, vss)
        single.cache_len.copy_(torch.where(active, single.cache_len, saved))
    torch.cuda.synchronize()
    want_len = [min(L, s + n_) for s, n_ in zip(start, lens)]
    assert bulk.cache_len.tolist() == want_len == single.cache_len.tolist()
    for a, b in ((bulk.k, single.k), (bulk.v, single.v), (bulk.k_scale, single.k_scale), (bulk.v_scale, single.v_scale)):
        assert torch.equal(a, b)
    assert torch.equal(bulk.k[0, 1, 16], k[16, d:2 * d]) and torch.equal(bulk.v[2, 2, 5], v[17, 2 * d:3 * d])
    assert not bulk.k[1].any()
