"""GPU: split-KV decode through the C ABI against the decode oracle (train/cpu_infer.cpp:413-460).

int8 QK^T accumulators must be bit-exact; outputs within max-abs 2e-2 / mean-abs 2e-3 of the
oracle on outputs rescaled to unit variance."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tests.common import assert_within_tolerance
from tscale_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=64, max_heads=16, max_head_dim=128, max_splits=32)
    yield c
    c.close()


def make_cache(seed, dtype, B, H, L, d, lens):
    rng = np.random.default_rng(seed)
    k = np.zeros((B, H, L, d), np.uint8); v = np.zeros_like(k)
    ks = np.zeros((B, H, L), np.float32); vs = np.zeros_like(ks)
    for b in range(B):
        n = lens[b]
        if n == 0:
            continue
        kq, kss = orc.quantize_rows(dtype, rng.standard_normal((n, H * d)).astype(np.float32), H)
        vq, vss = orc.quantize_rows(dtype, rng.standard_normal((n, H * d)).astype(np.float32), H)
        k[b, :, :n] = kq.reshape(n, H, d).transpose(1, 0, 2)
        v[b, :, :n] = vq.reshape(n, H, d).transpose(1, 0, 2)
        ks[b, :, :n] = kss; vs[b, :, :n] = vss
    return k, v, ks, vs


def gpu_cache(ctx, dtype, k, v, ks, vs, lens):
    from tscale_amd import KVCache
    B, H, L, d = k.shape
    c = KVCache(ctx, dtype, B, H, L, d)
    c.k.copy_(torch.from_numpy(k)); c.v.copy_(torch.from_numpy(v))
    c.k_scale.copy_(torch.from_numpy(ks)); c.v_scale.copy_(torch.from_numpy(vs))
    c.cache_len.copy_(torch.tensor(lens, dtype=torch.int32))
    return c


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("window,slope,splits", [(10 ** 6, 0.0, 0), (64, 0.5, 3), (0, 0.0, 1), (1, 0.3, 2), (700, 0.01, 8)])
def test_decode_parity_ragged(ctx, dtype, d, window, slope, splits):
    B, H, L = 5, 3, 1500
    lens = [1500, 1, 0, 777, 130]
    k, v, ks, vs = make_cache(100 + d, dtype, B, H, L, d, lens)
    rng = np.random.default_rng(7)
    q, qs = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
    qs = np.ascontiguousarray(qs.T)  # [B, H]
    want, want_acc = orc.decode(dtype, q, qs, k, v, ks, vs, np.array(lens, np.int32), window, slope, want_acc=True)
    cache = gpu_cache(ctx, dtype, k, v, ks, vs, lens)
    dbg = torch.zeros((B, H, L), dtype=torch.int32 if dtype == capi.I8 else torch.float32, device="cuda")
    out = ctx.compute_val_lookup_decode(cache, torch.from_numpy(q).cuda(), torch.from_numpy(qs).cuda(), window, slope,
                                        n_splits=splits, debug_qk_acc=dbg)
    torch.cuda.synchronize()
    out = out.cpu().numpy(); acc = dbg.cpu().numpy()
    for b, n in enumerate(lens):
        if n == 0:
            assert not out[b].any()
            continue
        lo, hi = (n - 1, n) if window == 0 else (max(0, n - 1 - window), n - 1)
        if dtype == capi.I8:
            assert np.array_equal(acc[b, :, lo:hi], want_acc[b, :, lo:hi]), "int32 QK^T accumulators differ"
        else:
            bound = 4 * 2.0 ** -23 * np.maximum(np.abs(want_acc[b, :, lo:hi]), 1.0) * 16
            assert np.all(np.abs(acc[b, :, lo:hi] - want_acc[b, :, lo:hi]) <= bound)
    assert_within_tolerance(out, want, "decode")
    assert np.abs(out - want).max() < 1e-4  # fp32 softmax on both sides: far inside the tolerance


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
def test_decode_bf16_query_is_quantised_like_the_oracle(ctx, dtype):
    B, H, L, d = 4, 2, 600, 128
    lens = [600, 31, 257, 512]
    k, v, ks, vs = make_cache(5, dtype, B, H, L, d, lens)
    qf = torch.randn((B, H * d), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    bits = qf.view(torch.int16).numpy().view(np.uint16)
    q8, qs = orc.quantize_rows(dtype, bits, H)
    want, want_acc = orc.decode(dtype, q8, np.ascontiguousarray(qs.T), k, v, ks, vs, np.array(lens, np.int32), 10 ** 6, 0.0,
                                want_acc=True)
    cache = gpu_cache(ctx, dtype, k, v, ks, vs, lens)
    dbg = torch.zeros((B, H, L), dtype=torch.int32 if dtype == capi.I8 else torch.float32, device="cuda")
    out = ctx.compute_val_lookup_decode(cache, qf.cuda(), None, 10 ** 6, 0.0, debug_qk_acc=dbg).cpu().numpy()
    if dtype == capi.I8:
        for b, n in enumerate(lens):
            assert np.array_equal(dbg.cpu().numpy()[b, :, :n - 1], want_acc[b, :, :n - 1])
    assert np.abs(out - want).max() < 1e-4


def test_decode_constant_scales_and_reference_polynomial(ctx):
    """TScale's own model: q and v scales are the constant VEC_SCALE = 1/24 (cpu_infer.cpp:16,448,454); the
    reference's polynomial exp2 stays within the tolerance of the kernel's v_exp_f32."""
    from tscale_amd import KVCache
    B, H, L, d = 2, 4, 900, 128
    lens = [900, 333]
    rng = np.random.default_rng(11)
    k = rng.integers(-127, 128, (B, H, L, d)).astype(np.int8).view(np.uint8)
    v = rng.integers(-127, 128, (B, H, L, d)).astype(np.int8).view(np.uint8)
    ks = (rng.random((B, H, L)).astype(np.float32) + 0.5) / 24 / 24
    q = rng.integers(-127, 128, (B, H * d)).astype(np.int8).view(np.uint8)
    VEC = 1.0 / 24
    want = orc.decode(orc.I8, q, VEC, k, v, ks, VEC, np.array(lens, np.int32), 64, 0.5, exp2_mode=1, use_simd=True)
    cache = KVCache(ctx, capi.I8, B, H, L, d)
    cache.k.copy_(torch.from_numpy(k)); cache.v.copy_(torch.from_numpy(v)); cache.k_scale.copy_(torch.from_numpy(ks))
    cache.v_scale = VEC
    cache.cache_len.copy_(torch.tensor(lens, dtype=torch.int32))
    out = ctx.compute_val_lookup_decode(cache, torch.from_numpy(q).cuda(), VEC, 64, 0.5).cpu().numpy()
    assert_within_tolerance(out, want, "decode vs polynomial-exp2 oracle")


def test_decode_full_size_properties(ctx):
    """The benchmark's decode shape (B64, L4096, H16, d128, int8, bf16 query): size-independent properties.
    (a) V = ones with scale 1 -> every output element equals 1 - 2^-swl >= 0 and is identical across d;
    (b) the result does not depend on the number of KV splits beyond fp32 re-association."""
    from tscale_amd import KVCache
    B, H, L, d = 64, 16, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(1)
    cache = KVCache(ctx, capi.I8, B, H, L, d)
    cache.k.copy_(torch.randint(0, 256, (B, H, L, d), dtype=torch.uint8, device="cuda", generator=g))
    cache.v.fill_(1)
    cache.k_scale.copy_(torch.rand((B, H, L), device="cuda", generator=g) * 0.01)
    cache.v_scale = 1.0
    cache.cache_len.fill_(L)
    q = torch.randn((B, H * d), device="cuda", generator=g).to(torch.bfloat16)
    outs = [ctx.compute_val_lookup_decode(cache, q, None, 10 ** 6, 0.0, n_splits=s).cpu().numpy() for s in (1, 4, 16)]
    o = outs[0].reshape(B, H, d)
    assert np.all(o >= 0) and np.all(o < 1) and np.abs(o - o[:, :, :1]).max() < 1e-6
    assert np.abs(outs[0] - outs[1]).max() < 1e-5 and np.abs(outs[0] - outs[2]).max() < 1e-5
    # (c) one (sequence, head) checked against the oracle at full length
    kq = cache.k[3:4, 5:6].cpu().numpy(); vq = cache.v[3:4, 5:6].cpu().numpy(); ksn = cache.k_scale[3:4, 5:6].cpu().numpy()
    bits = q[3:4, 5 * d:6 * d].cpu().view(torch.int16).numpy().view(np.uint16)
    q8, qs = orc.quantize_rows(orc.I8, bits, 1)
    want = orc.decode(orc.I8, q8, qs.T.copy(), kq, vq, ksn, 1.0, np.array([L], np.int32), 10 ** 6, 0.0)
    assert np.abs(outs[1][3, 5 * d:6 * d] - want[0]).max() < 1e-5


@pytest.mark.parametrize("seed", range(8))
def test_decode_randomised_shapes(ctx, seed):
    """Seeded random decode launches: batch, heads, cache capacity and lengths (empty, one row, full), windows, slopes,
    split counts (auto, 1, several), with and without the fused append; always against the oracle."""
    rng = np.random.default_rng(2000 + seed)
    dtype = [capi.I8, capi.E4M3][seed % 2]
    d = [128, 64][(seed // 2) % 2]
    B, H = int(rng.integers(1, 9)), int(rng.choice([1, 2, 3, 5, 8, 16]))
    L = int(rng.choice([8, 100, 513, 2000]))
    lens = [int(x) for x in rng.integers(0, L + 1, B)]
    lens[0] = L                      # one full cache
    if B > 1:
        lens[1] = 0                  # one empty
    window = int(rng.choice([1, 2, 64, 100, 10 ** 6])) if seed % 4 else 0
    slope = float(rng.choice([0.0, 0.3]))
    splits = int(rng.choice([0, 1, 2, 5]))
    k, v, ks, vs = make_cache(300 + seed, dtype, B, H, L, d, lens)
    q, qs = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
    qs = np.ascontiguousarray(qs.T)
    cache = gpu_cache(ctx, dtype, k, v, ks, vs, lens)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    what = f"seed {seed}: dtype {dtype} d {d} B {B} H {H} L {L} lens {lens} window {window} slope {slope} splits {splits}"
    if window == 0 or seed % 2 == 0:
        want = orc.decode(dtype, q, qs, k, v, ks, vs, np.array(lens, np.int32), window, slope)
        out = ctx.compute_val_lookup_decode(cache, dev(q), dev(qs), window, slope, n_splits=splits).cpu().numpy()
    else:
        # fused append of one new row per sequence; the oracle appends to its own copy first
        kq, kss = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
        vq, vss = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
        new_lens = []
        for b in range(B):
            n = lens[b]
            if n < L:
                k[b, :, n] = kq[b].reshape(H, d); v[b, :, n] = vq[b].reshape(H, d)
                ks[b, :, n] = kss[:, b]; vs[b, :, n] = vss[:, b]
                n += 1
            new_lens.append(n)
        want = orc.decode(dtype, q, qs, k, v, ks, vs, np.array(new_lens, np.int32), window, slope)
        out = ctx.compute_val_lookup_decode(cache, dev(q), dev(qs), window, slope, n_splits=splits,
                                            append=(dev(kq), dev(kss.T), dev(vq), dev(vss.T))).cpu().numpy()
        assert cache.cache_len.cpu().numpy().tolist() == new_lens, what
        assert np.array_equal(cache.k.cpu().numpy(), k) and np.array_equal(cache.k_scale.cpu().numpy(), ks), what
    assert np.abs(out - want).max() < 1e-4 * max(1.0, np.abs(want).max()), what


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("window,splits", [(10 ** 6, 1), (10 ** 6, 4), (64, 0), (0, 1), (1, 2)])
def test_decode_fused_kv_product_equals_the_separate_call(ctx, d, window, splits):
    """KVProduct written by the decode launches (one split: by the attention kernel; several: by the merge) is what
    tsattn_kv_product makes from the stored output, byte for byte, and what the oracle makes from it; sequences
    without keys give zeros."""
    B, H, L, rep = 5, 4, 300, 4
    lens = [300, 1, 17, 0, 129]
    rng = np.random.default_rng(d + window % 1000 + splits)
    k, v, ks, vs = make_cache(900 + d, capi.I8, B, H, L, d, lens)
    q, qs = orc.quantize_rows(capi.I8, rng.standard_normal((B, H * d)).astype(np.float32), H)
    cache = gpu_cache(ctx, capi.I8, k, v, ks, vs, lens)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    kvec = rng.integers(-127, 128, (B, H * d + 16)).astype(np.int8)          # the token's K vector, padded pitch
    dk = dev(kvec.view(np.uint8))[:, :H * d]
    kv = torch.full((B, H * rep * d + 32), 99, dtype=torch.uint8, device="cuda")
    mult = 0.75
    out = ctx.compute_val_lookup_decode(cache, dev(q), dev(np.ascontiguousarray(qs.T)), window, 0.25, n_splits=splits,
                                        kv_product=(dk, kv[:, :H * rep * d], rep, mult))
    torch.cuda.synchronize()
    want = ctx.kv_product(dk, out, H, rep, mult=mult).cpu().numpy()
    assert np.array_equal(kv[:, :H * rep * d].cpu().numpy(), want)
    assert (kv[:, H * rep * d:] == 99).all()
    assert np.array_equal(want.view(np.int8), orc.kv_product(kvec[:, :H * d], out.cpu().numpy(), H, rep, mult))
    assert not want[3].any()                                                   # the empty sequence
