"""GPU: the prompt-then-generate flow of the reference's CPU inference loop (gpt/train/cpu_infer.cpp:466-520,
586-600) restricted to its attention calls: prefill over the prompt, the prompt's K/V rows moved into the KV
cache, then one decode call per generated token after an append.  Every decode step is checked against the
decode oracle on the same cache, and against the prefill oracle's row of the same position (the property
the reference's own CPU/GPU check relies on, cpu_infer.cpp:658-683)."""
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


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("window,slope", [(10 ** 6, 0.0), (64, 0.5), (1, 0.0)])
def test_prompt_then_generate(ctx, dtype, window, slope):
    from tscale_amd import KVCache
    B, H, d = 3, 4, 128
    prompt = [150, 37, 96]
    n_new = 6
    total = [p + n_new for p in prompt]
    L = max(total) + 2
    rng = np.random.default_rng(11 + dtype)
    # all tokens of every sequence (prompt + generated) are drawn up front so that prefill over the whole
    # sequence is available as the second reference
    tot_off = np.concatenate([[0], np.cumsum(total)])
    n_all = int(tot_off[-1])
    q_all, qs_all = orc.quantize_rows(dtype, rng.standard_normal((n_all, H * d)).astype(np.float32), H)
    k_all, ks_all = orc.quantize_rows(dtype, rng.standard_normal((n_all, H * d)).astype(np.float32), H)
    v_all, vs_all = orc.quantize_rows(dtype, rng.standard_normal((n_all, H * d)).astype(np.float32), H)
    st, fi = orc.make_spans(total, window)
    want_prefill = orc.prefill_q8(dtype, q_all, k_all, v_all, H, qs_all, ks_all, vs_all, st, fi, slope)

    # prompt rows in prefill layout
    rows = np.concatenate([np.arange(tot_off[b], tot_off[b] + prompt[b]) for b in range(B)])
    p_off = np.concatenate([[0], np.cumsum(prompt)]).astype(np.int32)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    qp, kp, vp = dev(q_all[rows]), dev(k_all[rows]), dev(v_all[rows])
    qsp, ksp, vsp = dev(qs_all[:, rows]), dev(ks_all[:, rows]), dev(vs_all[:, rows])
    off_dev = dev(p_off)
    pst, pfi = ctx.build_spans(off_dev, len(rows), window)
    out_prompt = ctx.compute_val_lookup(dtype, H, qp, kp, vp, qsp, ksp, vsp, pst, pfi, slope).cpu().numpy()
    assert_within_tolerance(out_prompt, want_prefill[rows], "prompt prefill")

    cache = KVCache(ctx, dtype, B, H, L, d)
    cache.fill_from_prefill(off_dev, kp, ksp, vp, vsp)
    assert cache.cache_len.tolist() == prompt

    # host copy of the cache for the decode oracle
    hk = np.zeros((B, H, L, d), np.uint8); hv = np.zeros_like(hk)
    hks = np.zeros((B, H, L), np.float32); hvs = np.zeros_like(hks)
    for b in range(B):
        r = np.arange(tot_off[b], tot_off[b] + total[b])
        hk[b, :, :total[b]] = k_all[r].reshape(-1, H, d).transpose(1, 0, 2)
        hv[b, :, :total[b]] = v_all[r].reshape(-1, H, d).transpose(1, 0, 2)
        hks[b, :, :total[b]] = ks_all[:, r]; hvs[b, :, :total[b]] = vs_all[:, r]

    for step in range(n_new):
        cur = np.array([tot_off[b] + prompt[b] + step for b in range(B)])
        cache.add_vectors(dev(k_all[cur]), dev(ks_all[:, cur].T), dev(v_all[cur]), dev(vs_all[:, cur].T))
        lens = np.array([prompt[b] + step + 1 for b in range(B)], np.int32)
        assert cache.cache_len.tolist() == lens.tolist()
        q, qs = q_all[cur], np.ascontiguousarray(qs_all[:, cur].T)
        got = ctx.compute_val_lookup_decode(cache, dev(q), dev(qs), window, slope).cpu().numpy()
        want = orc.decode(dtype, q, qs, hk, hv, hks, hvs, lens, window, slope)
        assert np.abs(got - want).max() < 1e-4, f"step {step}"
        assert_within_tolerance(got, want_prefill[cur], f"decode step {step} vs prefill row")
    # the cache now holds exactly the rows the oracle saw
    torch.cuda.synchronize()
    for b in range(B):
        assert np.array_equal(cache.k[b, :, :total[b]].cpu().numpy(), hk[b, :, :total[b]])
        assert np.array_equal(cache.v_scale[b, :, :total[b]].cpu().numpy(), hvs[b, :, :total[b]])


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("window,slope,splits", [(10 ** 6, 0.0, 0), (64, 0.5, 1), (1, 0.0, 1), (10 ** 6, 0.1, 3)])
def test_fused_append_equals_append_then_decode(ctx, dtype, window, slope, splits):
    """tsattn_decode with k_new/v_new does what tsattn_cache_append + tsattn_decode do (cpu_infer.cpp:506-509):
    same cache contents, same lengths, bit-identical outputs, step after step; a full cache drops the row in
    both."""
    from tscale_amd import KVCache
    B, H, d, L = 4, 3, 128, 40
    start = [0, 17, 38, 5]          # sequence 2 fills up after two steps
    rng = np.random.default_rng(3)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    caches = []
    for _ in range(2):
        c = KVCache(ctx, dtype, B, H, L, d)
        caches.append(c)
    fill = rng.integers(0, 256, (B, H, L, d)).astype(np.uint8)
    if dtype == capi.E4M3:
        fill[(fill & 0x7f) == 0x7f] = 0x10   # no NaN codes
    sc = (rng.random((B, H, L)).astype(np.float32) + 0.5) / 24
    for c in caches:
        c.k.copy_(dev(fill)); c.v.copy_(dev(fill[::-1]))
        c.k_scale.copy_(dev(sc)); c.v_scale.copy_(dev(sc[:, ::-1]))
        c.cache_len.copy_(torch.tensor(start, dtype=torch.int32))
    for step in range(4):
        kq, ks = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
        vq, vs = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
        qq, qs = orc.quantize_rows(dtype, rng.standard_normal((B, H * d)).astype(np.float32), H)
        k_new, ks_new, v_new, vs_new = dev(kq), dev(ks.T), dev(vq), dev(vs.T)
        q, q_s = dev(qq), dev(qs.T)
        caches[0].add_vectors(k_new, ks_new, v_new, vs_new)
        want = ctx.compute_val_lookup_decode(caches[0], q, q_s, window, slope, n_splits=splits)
        got = ctx.compute_val_lookup_decode(caches[1], q, q_s, window, slope, n_splits=splits,
                                            append=(k_new, ks_new, v_new, vs_new))
        torch.cuda.synchronize()
        assert caches[0].cache_len.tolist() == caches[1].cache_len.tolist() == [min(L, s + step + 1) for s in start]
        assert torch.equal(got, want), f"step {step}"
        for a, b in ((caches[0].k, caches[1].k), (caches[0].v, caches[1].v), (caches[0].k_scale, caches[1].k_scale),
                     (caches[0].v_scale, caches[1].v_scale)):
            assert torch.equal(a, b)
    # window 0 is refused for the fused form
    with pytest.raises(capi.TsattnError):
        ctx.compute_val_lookup_decode(caches[1], q, q_s, 0, 0.0, append=(k_new, ks_new, v_new, vs_new))


def test_single_split_writes_the_output_directly(ctx):
    """With one split there is no merge launch; the result equals the multi-split one up to summation order."""
    B, H, d, L = 6, 4, 128, 900
    rng = np.random.default_rng(9)
    from tscale_amd import KVCache
    c = KVCache(ctx, capi.I8, B, H, L, d)
    lens = [900, 1, 0, 333, 64, 2]
    hk = np.zeros((B, H, L, d), np.uint8); hv = np.zeros_like(hk)
    hks = np.zeros((B, H, L), np.float32); hvs = np.zeros_like(hks)
    for b, n in enumerate(lens):
        if n:
            kq, kss = orc.quantize_rows(orc.I8, rng.standard_normal((n, H * d)).astype(np.float32), H)
            vq, vss = orc.quantize_rows(orc.I8, rng.standard_normal((n, H * d)).astype(np.float32), H)
            hk[b, :, :n] = kq.reshape(n, H, d).transpose(1, 0, 2); hv[b, :, :n] = vq.reshape(n, H, d).transpose(1, 0, 2)
            hks[b, :, :n] = kss; hvs[b, :, :n] = vss
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    c.k.copy_(dev(hk)); c.v.copy_(dev(hv)); c.k_scale.copy_(dev(hks)); c.v_scale.copy_(dev(hvs))
    c.cache_len.copy_(torch.tensor(lens, dtype=torch.int32))
    q, qs = orc.quantize_rows(orc.I8, rng.standard_normal((B, H * d)).astype(np.float32), H)
    qs = np.ascontiguousarray(qs.T)
    want = orc.decode(orc.I8, q, qs, hk, hv, hks, hvs, np.array(lens, np.int32), 10 ** 6, 0.0)
    one = ctx.compute_val_lookup_decode(c, dev(q), dev(qs), 10 ** 6, 0.0, n_splits=1).cpu().numpy()
    many = ctx.compute_val_lookup_decode(c, dev(q), dev(qs), 10 ** 6, 0.0, n_splits=5).cpu().numpy()
    assert np.abs(one - want).max() < 1e-4 and np.abs(many - want).max() < 1e-4
    assert not one[2].any() and not one[1].any()      # no keys: exact zeros
