"""GPU: one layer of the int8 inference path, token by token (tscale_amd.attention.add_lookup_product: a chain of
library calls through the C ABI) against the oracle's AddLookupProduct (gpt/train/cpu_infer.cpp:465-527).  Each step
starts from the state the GPU path holds, so inputs are identical: appended cache rows and key scales must be the same
bytes, the attention output agrees to a few ulps, the new state is the same up to flips of single int8 roundings."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tscale_amd import KVCache, capi
from tscale_amd.attention import VEC_SCALE, add_lookup_product, flush_state

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=8, max_heads=4, max_head_dim=128)
    yield c
    c.close()


@pytest.mark.parametrize("H,d,dim,width,slope,relu_dim", [
    (2, 128, 256, 1000, 0.0, 256), (4, 64, 512, 3, 0.5, 256), (2, 128, 384, 0, 0.0, 256),
    # feed-forward groups of 128 * ReluMult (model_dim.h:66): ReluMult 2, 3 and 4
    (2, 128, 256, 1000, 0.0, 512), (3, 128, 384, 5, 0.5, 3 * 384), (2, 64, 256, 2, 0.0, 2 * 512)])
def test_layer_steps_match_the_oracle(ctx, H, d, dim, width, slope, relu_dim):
    B, max_len, steps = 4, 12, 6
    qsum = H * d
    rng = np.random.default_rng(H * d + width)
    mat = lambda n, k: np.clip(np.rint(rng.standard_normal((n, k)) * 32), -127, 127).astype(np.int8)
    mats = {"qk": mat(qsum, dim), "qv": mat(qsum, dim), "k": mat(qsum, dim), "v": mat(qsum, dim),
            "combiner": mat(dim, qsum * 4), "expand": mat(relu_dim, dim), "contract": mat(dim, relu_dim)}
    scales = (0.031, 0.027, 0.035)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    layer = {"proj": dev(np.concatenate([mats[n] for n in ("qk", "qv", "k", "v")]).view(np.uint8)),
             "combiner": dev(mats["combiner"].view(np.uint8)), "expand": dev(mats["expand"].view(np.uint8)),
             "contract": dev(mats["contract"].view(np.uint8)), "qv_scale": scales[0], "combiner_scale": scales[1],
             "contract_scale": scales[2], "width": width, "slope": slope}
    # caches with some history; sequence 3 runs into the end of its cache
    # (values in [-127, 127] as the reference's conversion leaves them: its vpdpbusd dot product, which the oracle
    # follows, is not defined for -128, cpu_infer.cpp:88-92)
    kc = rng.integers(-127, 128, (B, H, max_len, d)).astype(np.int8).view(np.uint8)
    vc = rng.integers(-127, 128, (B, H, max_len, d)).astype(np.int8).view(np.uint8)
    ksc = ((rng.random((B, H, max_len)) + 0.5) * 1e-3).astype(np.float32)
    lens = np.array([0, 2, 7, 9], dtype=np.int32)
    cache = KVCache(ctx, capi.I8, B, H, max_len, d)
    cache.k.copy_(dev(kc)); cache.v.copy_(dev(vc)); cache.k_scale.copy_(dev(ksc)); cache.v_scale.fill_(VEC_SCALE)
    cache.cache_len.copy_(dev(lens))
    rope_np = orc.fill_rope(d, 64)
    rope = dev(rope_np)
    state = dev(rng.standard_normal((B, dim)).astype(np.float32) * 2)
    room = torch.empty(16 * 4 * B * dim, dtype=torch.uint8, device="cuda")
    keep = {}
    exact_steps = 0
    for step in range(steps):
        t = (lens + 3).astype(np.int32)
        st_in = state.cpu().numpy()
        want, want_val = orc.add_lookup_product(mats, scales, width, slope, H, d, t, rope_np, st_in, kc, vc, ksc, lens)
        val = add_lookup_product(ctx, layer, cache, dev(t), rope, state, workspace=room, scratch=keep)
        torch.cuda.synchronize()
        assert cache.cache_len.cpu().numpy().tolist() == lens.tolist()
        assert np.array_equal(cache.k.cpu().numpy(), kc) and np.array_equal(cache.v.cpu().numpy(), vc), f"step {step}: cache rows"
        assert np.array_equal(cache.k_scale.cpu().numpy(), ksc), f"step {step}: cached key scales"
        assert np.abs(val.cpu().numpy() - want_val).max() < 2e-5
        got = state.cpu().numpy()
        rms = np.sqrt((want.astype(np.float64) ** 2).mean())
        assert np.abs(got - want).max() / rms < 2e-2, f"step {step}"
        exact_steps += int(np.array_equal(got, want))
    assert lens.tolist() == [min(max_len, l + steps) for l in (0, 2, 7, 9)]
    assert exact_steps >= steps // 2, "most steps come out bit-identical"


@pytest.mark.parametrize("width,slope", [(1000, 0.0), (16, 0.5)])
def test_prompt_layer_equals_the_oracle_token_by_token(ctx, width, slope):
    """A batch of prompt tokens through add_lookup_product_prompt (one prefill launch, one cache fill) against the oracle
    fed one token at a time: same cache bytes and key scales, attention output within the prefill tolerance, states the
    same up to flips of int8 roundings."""
    from tscale_amd.attention import add_lookup_product_prompt
    H, d, dim, max_len = 2, 128, 256, 64
    seq_lens = [37, 50, 1]
    B, n = len(seq_lens), sum(seq_lens)
    qsum = H * d
    rng = np.random.default_rng(width)
    mat = lambda r, k: np.clip(np.rint(rng.standard_normal((r, k)) * 32), -127, 127).astype(np.int8)
    mats = {"qk": mat(qsum, dim), "qv": mat(qsum, dim), "k": mat(qsum, dim), "v": mat(qsum, dim),
            "combiner": mat(dim, qsum * 4), "expand": mat(qsum, dim), "contract": mat(dim, qsum)}
    scales = (0.031, 0.027, 0.035)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    layer = {"proj": dev(np.concatenate([mats[m] for m in ("qk", "qv", "k", "v")]).view(np.uint8)),
             "combiner": dev(mats["combiner"].view(np.uint8)), "expand": dev(mats["expand"].view(np.uint8)),
             "contract": dev(mats["contract"].view(np.uint8)), "qv_scale": scales[0], "combiner_scale": scales[1],
             "contract_scale": scales[2], "width": width, "slope": slope}
    rope_np = orc.fill_rope(d, max_len)
    state0 = rng.standard_normal((n, dim)).astype(np.float32) * 2
    # oracle: every sequence on its own, token after token
    kc = np.zeros((B, H, max_len, d), dtype=np.uint8); vc = np.zeros_like(kc)
    ksc = np.zeros((B, H, max_len), dtype=np.float32)
    want = np.empty_like(state0); want_val = np.empty((n, qsum), dtype=np.float32)
    off = np.concatenate([[0], np.cumsum(seq_lens)])
    for b in range(B):
        lens = np.zeros(1, dtype=np.int32)
        for p_ in range(seq_lens[b]):
            tok = off[b] + p_
            o, v_ = orc.add_lookup_product(mats, scales, width, slope, H, d, np.array([p_], dtype=np.int32), rope_np,
                                           state0[tok:tok + 1], kc[b:b + 1], vc[b:b + 1], ksc[b:b + 1], lens)
            want[tok], want_val[tok] = o[0], v_[0]
    # GPU: the whole batch at once
    cache = KVCache(ctx, capi.I8, B, H, max_len, d)
    cache.v_scale.fill_(VEC_SCALE)
    seq_offset = dev(off.astype(np.int32))
    pos = dev(np.concatenate([np.arange(l) for l in seq_lens]).astype(np.int32))
    st, fi = ctx.build_spans(seq_offset, n, width)
    state = dev(state0)
    val = add_lookup_product_prompt(ctx, layer, cache, seq_offset, pos, dev(rope_np), state, st, fi)
    torch.cuda.synchronize()
    assert cache.cache_len.cpu().numpy().tolist() == seq_lens
    assert np.array_equal(cache.k.cpu().numpy(), kc) and np.array_equal(cache.v.cpu().numpy(), vc)
    assert np.array_equal(cache.k_scale.cpu().numpy(), ksc)
    from tests.common import assert_within_tolerance
    assert_within_tolerance(val.cpu().numpy(), want_val, "attention output of the prompt")
    got = state.cpu().numpy()
    rms = np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.abs(got - want).max() / rms < 5e-2
    assert np.sqrt(((got - want).astype(np.float64) ** 2).mean()) / rms < 5e-3


def test_deferred_state_updates_give_the_same_bits(ctx):
    """Three layers, three tokens: each layer's last state update left to the next layer's first normalisation (and to
    flush_state after the last) gives the same states, cache rows and attention outputs as updating at once."""
    B, H, d, dim, max_len = 4, 2, 128, 256, 8
    qsum = H * d
    rng = np.random.default_rng(77)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    mat = lambda n, k: dev(np.clip(np.rint(rng.standard_normal((n, k)) * 32), -127, 127).astype(np.int8).view(np.uint8))
    layers = [{"proj": mat(4 * qsum, dim), "combiner": mat(dim, qsum * 4), "expand": mat(qsum, dim), "contract": mat(dim, qsum),
               "qv_scale": 0.031, "combiner_scale": 0.027, "contract_scale": 0.035, "width": w, "slope": s}
              for w, s in ((1, 0.0), (0, 0.0), (1000, 0.5))]
    rope = dev(orc.fill_rope(d, 64))
    start = rng.standard_normal((B, dim)).astype(np.float32) * 2
    results = []
    for defer in (False, True):
        caches = [KVCache(ctx, capi.I8, B, H, max_len, d) for _ in layers]
        for c in caches:
            c.k.zero_(); c.v.zero_(); c.k_scale.zero_(); c.v_scale.fill_(VEC_SCALE); c.cache_len.zero_()
        state = dev(start)
        keep, vals = {}, []
        for step in range(3):
            t = torch.full((B,), step, dtype=torch.int32, device="cuda")
            pending = None
            for layer, c in zip(layers, caches):
                if defer:
                    val, pending = add_lookup_product(ctx, layer, c, t, rope, state, scratch=keep, pending=pending, defer=True)
                else:
                    val = add_lookup_product(ctx, layer, c, t, rope, state, scratch=keep)
                vals.append(val.cpu().numpy().copy())
            if defer:
                norm = flush_state(ctx, pending, state)
                want_norm, _ = ctx.rope_normalize_rows(state, dim // 128, capi.I8)
                assert torch.equal(norm, want_norm)
        torch.cuda.synchronize()
        results.append((state.cpu().numpy(), [c.k.cpu().numpy() for c in caches], [c.k_scale.cpu().numpy() for c in caches], vals))
    a, b = results
    assert np.array_equal(a[0], b[0])
    for x, y in zip(a[1] + a[2] + a[3], b[1] + b[2] + b[3]):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("width,slope", [(64, 0.5), (10 ** 6, 0.0)])
def test_prompt_form_equals_token_form_at_model_width(ctx, width, slope):
    """At the 1.5B-style width (2048, 16 heads of 128): 32 sequences of 128 tokens through the prompt form of the layer
    (products of 4096 rows: the large-tile kernels, the producer's 32-pair launches, one prefill launch, one cache
    fill) and the same tokens one position at a time through the token form (few-row products, fused append +
    attention + KVProduct): the same cache bytes and key scales, attention outputs within the prefill tolerance,
    states equal up to flips of int8 roundings -- the comparison NCPUInfer::Check makes (cpu_infer.cpp:658-683)."""
    from tests.common import assert_within_tolerance
    from tscale_amd import AttentionContext
    from tscale_amd.attention import add_lookup_product_prompt
    H, d, dim, B, S = 16, 128, 2048, 32, 128
    qsum, n = H * d, B * S
    big = AttentionContext(0, max_seqs=B, max_heads=H, max_head_dim=d)
    try:
        g = torch.Generator(device="cuda"); g.manual_seed(width % 1000)
        mat = lambda r, k: (torch.randn((r, k), device="cuda", generator=g) * 32).round().clamp(-127, 127).to(torch.int8).view(torch.uint8)
        layer = {"proj": mat(4 * qsum, dim), "combiner": mat(dim, qsum * 4), "expand": mat(qsum, dim), "contract": mat(dim, qsum),
                 "qv_scale": 0.031, "combiner_scale": 0.027, "contract_scale": 0.035, "width": width, "slope": slope}
        rope = torch.from_numpy(orc.fill_rope(d, S)).cuda()
        state0 = torch.randn((n, dim), device="cuda", generator=g) * 2          # token (b, p) at row b * S + p
        # prompt form
        c1 = KVCache(big, capi.I8, B, H, S, d); c1.v_scale.fill_(VEC_SCALE)
        seq_offset = torch.arange(0, n + 1, S, dtype=torch.int32, device="cuda")
        pos = torch.arange(S, dtype=torch.int32, device="cuda").repeat(B)
        st, fi = big.build_spans(seq_offset, n, min(width, S))
        s1 = state0.clone()
        v1 = add_lookup_product_prompt(big, layer, c1, seq_offset, pos, rope, s1, st, fi)
        # token form: position p of every sequence at step p
        c2 = KVCache(big, capi.I8, B, H, S, d); c2.v_scale.fill_(VEC_SCALE)
        s2 = state0.view(B, S, dim).transpose(0, 1).contiguous()                  # [S, B, dim]
        v2 = torch.empty((S, B, qsum), dtype=torch.float32, device="cuda")
        keep = {}
        for p_ in range(S):
            t = torch.full((B,), p_, dtype=torch.int32, device="cuda")
            v2[p_] = add_lookup_product(big, layer, c2, t, rope, s2[p_], scratch=keep)
        torch.cuda.synchronize()
        assert torch.equal(c1.cache_len, c2.cache_len) and int(c1.cache_len[0]) == S
        assert torch.equal(c1.k, c2.k) and torch.equal(c1.v, c2.v) and torch.equal(c1.k_scale, c2.k_scale)
        a_val = v1.view(B, S, qsum).transpose(0, 1).cpu().numpy().reshape(n, qsum)
        assert_within_tolerance(a_val, v2.cpu().numpy().reshape(n, qsum), "attention output, prompt form against token form")
        got = s1.view(B, S, dim).transpose(0, 1).cpu().numpy().astype(np.float64)
        want = s2.cpu().numpy().astype(np.float64)
        rms = np.sqrt((want ** 2).mean())
        assert np.abs(got - want).max() / rms < 5e-2
        assert np.sqrt(((got - want) ** 2).mean()) / rms < 5e-3
    finally:
        big.close()


def test_chained_prompt_layers_give_the_same_bits(ctx):
    """Two layers over a prompt of 4096 tokens (products large enough to normalise their own tiles): handing the second
    layer the normalised state the first layer's last product made gives the same bits as normalising afresh."""
    from tscale_amd import AttentionContext
    from tscale_amd.attention import add_lookup_product_prompt
    H, d, dim, B, S = 4, 128, 1024, 8, 512
    qsum, n = H * d, B * S
    big = AttentionContext(0, max_seqs=B, max_heads=H, max_head_dim=d)
    try:
        g = torch.Generator(device="cuda"); g.manual_seed(5)
        mat = lambda r, k: (torch.randn((r, k), device="cuda", generator=g) * 32).round().clamp(-127, 127).to(torch.int8).view(torch.uint8)
        layers = [{"proj": mat(4 * qsum, dim), "combiner": mat(dim, qsum * 4), "expand": mat(qsum, dim), "contract": mat(dim, qsum),
                   "qv_scale": 0.031, "combiner_scale": 0.027, "contract_scale": 0.035, "width": w, "slope": sl} for w, sl in ((64, 0.5), (10 ** 6, 0.0))]
        rope = torch.from_numpy(orc.fill_rope(d, S)).cuda()
        state0 = torch.randn((n, dim), device="cuda", generator=g) * 2
        seq_offset = torch.arange(0, n + 1, S, dtype=torch.int32, device="cuda")
        pos = torch.arange(S, dtype=torch.int32, device="cuda").repeat(B)
        results = []
        for chained in (False, True):
            state = state0.clone()
            caches = [KVCache(big, capi.I8, B, H, S, d) for _ in layers]
            norm = None
            for layer, c in zip(layers, caches):
                c.v_scale.fill_(VEC_SCALE)
                st, fi = big.build_spans(seq_offset, n, min(layer["width"], S))
                if chained:
                    _, norm = add_lookup_product_prompt(big, layer, c, seq_offset, pos, rope, state, st, fi, norm=norm, want_norm=True)
                else:
                    add_lookup_product_prompt(big, layer, c, seq_offset, pos, rope, state, st, fi)
            torch.cuda.synchronize()
            if chained:
                want_norm, _ = big.rope_normalize_rows(state, dim // 128, capi.I8)
                assert torch.equal(norm, want_norm)
            results.append((state, [c.k for c in caches], [c.k_scale for c in caches]))
        assert torch.equal(results[0][0], results[1][0])
        for x, y in zip(results[0][1] + results[0][2], results[1][1] + results[1][2]):
            assert torch.equal(x, y)
    finally:
        big.close()
