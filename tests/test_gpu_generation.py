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
