"""GPU: the attention calls of the random-init 1.5B-style generation run at their real shapes (24 layers on the InitAlibi
schedule, gpt/model_params/model_dim.cpp:55-97; 16 heads of 128, int8, per-row scales; batch 32; a 2048-token prompt, then
tokens at cache lengths 2049...; the reference's loop is gpt/train/cpu_infer.cpp:466-520, 586-600).

Prefill over the prompt, once per distinct (width, slope) of the schedule: the size-independent property (V = ones gives
out = 1 - 2^-sum_weight_log in every column, first rows of sequences are zero) on the whole launch, and whole (sequence,
head) pairs against the oracle.  Then the fused append + decode on 24 caches for four tokens, sampled (layer, sequence, head)
pairs against the decode oracle on the same cache rows."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tests.common import assert_within_tolerance
from tscale_amd import capi
from tscale_amd.attention import alibi_layer_schedule

pytestmark = pytest.mark.gpu

B, S, H, D, DEPTH, NEW = 32, 2048, 16, 128, 24, 256
L = S + NEW


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=B, max_heads=H, max_head_dim=D, max_splits=32)
    yield c
    c.close()


def test_schedule_of_the_run():
    sched = alibi_layer_schedule(DEPTH, L)
    assert len(sched) == DEPTH and sorted(set(sched)) == [(1, 0.0), (64, 0.5), (L, 0.0)]
    assert sched[:4] == [(1, 0.0)] * 4 and sched[4:6] == [(64, 0.5), (L, 0.0)]


@pytest.mark.parametrize("window,slope", sorted(set(alibi_layer_schedule(DEPTH, L))))
def test_prompt_pass_attention_at_full_shape(ctx, window, slope):
    n = B * S
    g = torch.Generator(device="cuda").manual_seed(1313 + 5)
    q, qs = ctx.quantize_rows(torch.randn((n, H * D), device="cuda", generator=g), H, capi.I8)
    k, ks = ctx.quantize_rows(torch.randn((n, H * D), device="cuda", generator=g), H, capi.I8)
    v, vs = ctx.quantize_rows(torch.randn((n, H * D), device="cuda", generator=g), H, capi.I8)
    off = torch.arange(0, n + 1, S, dtype=torch.int32, device="cuda")
    st, fi = ctx.build_spans(off, n, window)
    # (a) the property, whole launch: V = 1 with scale 1
    ones = torch.ones((n, H * D), dtype=torch.uint8, device="cuda")
    swl = torch.zeros((H, n), device="cuda")
    out = ctx.compute_val_lookup(capi.I8, H, q, k, ones, qs, ks, 1.0, st, fi, slope, sum_weight_log=swl, causal_period=S)
    o = out.view(n, H, D)
    assert (o[::S] == 0).all()
    want = 1 - torch.exp2(-swl).t()
    assert (o - want[:, :, None]).abs().max().item() < 2e-3
    assert (o.max(dim=2).values - o.min(dim=2).values).max().item() < 1e-6
    del out, o, ones
    # (b) whole (sequence, head) pairs against the oracle, real V
    out = ctx.compute_val_lookup(capi.I8, H, q, k, v, qs, ks, vs, st, fi, slope, causal_period=S)
    st1, fi1 = orc.make_spans([S], window)
    for seq, head in ((0, 0), (17, 9), (31, 15)):
        rows, cols = slice(seq * S, (seq + 1) * S), slice(head * D, (head + 1) * D)
        cpu = lambda t: np.ascontiguousarray(t.cpu().numpy())
        want = orc.prefill_q8(orc.I8, cpu(q[rows, cols]), cpu(k[rows, cols]), cpu(v[rows, cols]), 1, cpu(qs[head:head + 1, rows]),
                              cpu(ks[head:head + 1, rows]), cpu(vs[head:head + 1, rows]), st1, fi1, slope)
        assert_within_tolerance(cpu(out[rows, cols]), want, f"prompt pass, window {window}, sequence {seq}, head {head}")


def test_generated_tokens_attention_at_full_shape(ctx):
    """Four tokens after the prompt through all 24 layers' attention: one cache per layer holding 2048 rows per sequence,
    the new token's K/V row appended by the decode call itself."""
    from tscale_amd import KVCache
    sched = alibi_layer_schedule(DEPTH, L)
    g = torch.Generator(device="cuda").manual_seed(77)
    caches = []
    for _ in range(DEPTH):
        c = KVCache(ctx, capi.I8, B, H, L, D)
        c.k[:, :, :S].copy_(torch.randint(-127, 128, (B, H, S, D), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8))
        c.v[:, :, :S].copy_(torch.randint(-127, 128, (B, H, S, D), dtype=torch.int8, device="cuda", generator=g).view(torch.uint8))
        c.k_scale[:, :, :S].copy_((torch.rand((B, H, S), device="cuda", generator=g) + 0.5) * 2e-3)
        c.v_scale[:, :, :S].copy_((torch.rand((B, H, S), device="cuda", generator=g) + 0.5) / 24)
        c.cache_len.fill_(S)
        caches.append(c)
    rng = np.random.default_rng(3)
    cpu = lambda t: np.ascontiguousarray(t.cpu().numpy())
    for step in range(4):
        for layer, (window, slope) in enumerate(sched):
            c = caches[layer]
            x = torch.randn((3, B, H * D), device="cuda", generator=g)
            q, qs = ctx.quantize_rows(x[0], H, capi.I8)
            kn, kns = ctx.quantize_rows(x[1], H, capi.I8)
            vn, vns = ctx.quantize_rows(x[2], H, capi.I8)
            qs, kns, vns = (s.t().contiguous() for s in (qs, kns, vns))   # [B, H]
            out = ctx.compute_val_lookup_decode(c, q, qs, window, slope, append=(kn, kns * 0.05, vn, vns))
            assert int(c.cache_len.min()) == int(c.cache_len.max()) == S + step + 1
            if layer in (0, 4, 5, 22, 23):
                for _ in range(2):
                    seq, head = int(rng.integers(0, B)), int(rng.integers(0, H))
                    n = S + step + 1
                    cols = slice(head * D, (head + 1) * D)
                    want = orc.decode(orc.I8, cpu(q[seq:seq + 1, cols]), cpu(qs[seq:seq + 1, head:head + 1]),
                                      cpu(c.k[seq:seq + 1, head:head + 1, :n]), cpu(c.v[seq:seq + 1, head:head + 1, :n]),
                                      cpu(c.k_scale[seq:seq + 1, head:head + 1, :n]), cpu(c.v_scale[seq:seq + 1, head:head + 1, :n]),
                                      np.array([n], np.int32), window, slope)
                    got = cpu(out[seq, cols])
                    assert np.abs(got - want[0]).max() < 1e-4 * max(1.0, np.abs(want).max()), (step, layer, seq, head)
                    # the appended row is the new token's
                    assert torch.equal(c.k[seq, head, n - 1], kn[seq, cols]) and torch.equal(c.v[seq, head, n - 1], vn[seq, cols])
