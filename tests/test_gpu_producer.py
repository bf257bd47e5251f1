"""GPU: the producer kernel (RoPE + per-head RMS normalisation + 8-bit conversion, tsattn_rope_normalize_rows)
through the C ABI against its oracle (gpt/att/rope.cpp:28-46, gpt/train/cpu_infer.cpp:358-391,486-499).
The kernel keeps the CPU path's operation order, so bytes and scales must be identical, not merely close."""
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
@pytest.mark.parametrize("d,H", [(64, 12), (128, 5)])
@pytest.mark.parametrize("with_rope", [True, False])
def test_producer_bit_exact(ctx, dtype, d, H, with_rope):
    n = 333                                     # (row, head) pairs not a multiple of the kernel's 64
    rng = np.random.default_rng(d + H)
    x = (rng.standard_normal((n, H * d)) * rng.uniform(0.05, 20, (n, 1))).astype(np.float32)
    x[7] = 0                                    # a zero row: zeros and scale 0
    x[9, d:2 * d] = 0                           # a zero head
    pos = rng.integers(0, 900, n).astype(np.int32) if with_rope else None
    rope_dev = ctx.fill_rope_table(d, 900)
    rope = orc.fill_rope(d, 900)
    assert np.array_equal(rope_dev.cpu().numpy(), rope)
    want_q, want_s = orc.rope_normalize_rows(dtype, x, H, pos=pos, rope=rope if with_rope else None, scale_mult=0.4)
    q, s = ctx.rope_normalize_rows(torch.from_numpy(x).cuda(), H, dtype,
                                   pos=None if pos is None else torch.from_numpy(pos).cuda(),
                                   rope=rope_dev if with_rope else None, scale_mult=0.4)
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy(), want_s)
    assert np.array_equal(q.cpu().numpy(), want_q)
    assert not q.cpu().numpy()[7].any() and s.cpu().numpy()[1, 9] == 0


@pytest.mark.parametrize("group", [256, 384, 512])
@pytest.mark.parametrize("n", [5, 700])
def test_producer_wide_groups_bit_exact(ctx, group, n):
    """The feed-forward groups of 128 * ReluMult (NormalizeState(relu, headCount), cpu_infer.cpp:519-524): int32 sums in
    two planes, ReLU on the int8 result; rotation and e4m3 are refused for such groups."""
    H = 3
    rng = np.random.default_rng(group + n)
    a = rng.integers(-20000, 20000, (n, H * group)).astype(np.int32)
    b = rng.integers(-20000, 20000, (n, H * group)).astype(np.int32)
    a[2, group:2 * group] = -b[2, group:2 * group]           # a group of zeros
    want_q, want_s = orc.rope_normalize_rows(orc.I8, a + b, H)
    want_q = np.where(want_q.view(np.int8) < 0, 0, want_q.view(np.int8)).astype(np.int8).view(np.uint8)
    planes = torch.from_numpy(np.stack([a, b])).cuda()
    q, s = ctx.rope_normalize_rows(planes, H, capi.I8, relu=True)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy(), want_q) and np.array_equal(s.cpu().numpy(), want_s)
    assert not q.cpu().numpy()[2, group:2 * group].any()
    x = torch.from_numpy((a + b).astype(np.float32)).cuda()
    with pytest.raises(capi.TsattnError):
        ctx.rope_normalize_rows(x, H, capi.E4M3)
    with pytest.raises(capi.TsattnError):
        ctx.rope_normalize_rows(x, H, capi.I8, pos=torch.zeros(n, dtype=torch.int32, device="cuda"), rope=ctx.fill_rope_table(128, 4))


def test_producer_int32_source_reverse_direction_and_clamped_positions(ctx):
    H, d, n = 4, 128, 70
    rng = np.random.default_rng(1)
    xi = rng.integers(-30000, 30000, (n, H * d)).astype(np.int32)
    rope = orc.fill_rope(d, 50)
    pos = rng.integers(-5, 80, n).astype(np.int32)              # out of range on both sides: clamped
    want_q, want_s = orc.rope_normalize_rows(orc.I8, xi, H, pos=np.clip(pos, 0, 49), rope=rope, rotate_dir=-1.0)
    q, s = ctx.rope_normalize_rows(torch.from_numpy(xi).cuda(), H, capi.I8, pos=torch.from_numpy(pos).cuda(),
                                   rope=torch.from_numpy(rope).cuda(), rotate_dir=-1.0)
    assert np.array_equal(q.cpu().numpy(), want_q) and np.array_equal(s.cpu().numpy(), want_s)


def test_producer_feeds_prefill(ctx):
    """Projection results -> producer -> prefill, all on the GPU, against the oracle's producer -> oracle's prefill:
    the reference's order of operations in AddLookupProduct (cpu_infer.cpp:479-509) for a whole sequence."""
    H, d = 4, 128
    seq_lens = [200, 120]
    n = sum(seq_lens)
    rng = np.random.default_rng(2)
    src = [rng.standard_normal((n, H * d)).astype(np.float32) * 3 for _ in range(3)]
    pos = np.concatenate([np.arange(L) for L in seq_lens]).astype(np.int32)
    rope = orc.fill_rope(d, 256)
    key_mult = 0.8 / 24 * np.float32(1.0 / np.sqrt(H * d))     # QVScale * VEC_SCALE * CalcDotScale(dim)
    oq, _ = orc.rope_normalize_rows(orc.I8, src[0], H, pos=pos, rope=rope)
    ok, oks = orc.rope_normalize_rows(orc.I8, src[1], H, pos=pos, rope=rope, scale_mult=key_mult)
    ov, _ = orc.rope_normalize_rows(orc.I8, src[2], H)
    st, fi = orc.make_spans(seq_lens, 10 ** 6)
    VEC = 1.0 / 24
    want = orc.prefill_q8(orc.I8, oq, ok, ov, H, VEC, oks, VEC, st, fi, 0.0)

    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    rope_dev = ctx.fill_rope_table(d, 256)
    gq, _ = ctx.rope_normalize_rows(dev(src[0]), H, capi.I8, pos=dev(pos), rope=rope_dev)
    gk, gks = ctx.rope_normalize_rows(dev(src[1]), H, capi.I8, pos=dev(pos), rope=rope_dev, scale_mult=key_mult)
    gv, _ = ctx.rope_normalize_rows(dev(src[2]), H, capi.I8)
    assert np.array_equal(gk.cpu().numpy(), ok) and np.array_equal(gks.cpu().numpy(), oks)
    off = dev(np.concatenate([[0], np.cumsum(seq_lens)]).astype(np.int32))
    gst, gfi = ctx.build_spans(off, n, 10 ** 6)
    out = ctx.compute_val_lookup(capi.I8, H, gq, gk, gv, VEC, gks, VEC, gst, gfi, 0.0).cpu().numpy()
    assert_within_tolerance(out, want, "producer -> prefill")


@pytest.mark.parametrize("d,H", [(64, 12), (128, 3)])
@pytest.mark.parametrize("f16", [False, True])
def test_kv_product_bit_exact(ctx, d, H, f16):
    """tsattn_kv_product against KVProduct of cpu_infer.cpp:320-337 on the same inputs: identical bytes."""
    n = 77
    rng = np.random.default_rng(d)
    k = rng.integers(-127, 128, (n, H * d)).astype(np.int8)
    val = (rng.standard_normal((n, H * d)) * 0.4).astype(np.float32)
    if f16:
        val = val.astype(np.float16).astype(np.float32)      # what the kernel sees when the attention output is half
    for mult in (1.0, 0.73):
        want = orc.kv_product(k, val, H, mult=mult)
        tv = torch.from_numpy(val).cuda()
        got = ctx.kv_product(torch.from_numpy(k.view(np.uint8)).cuda(), tv.half() if f16 else tv, H, mult=mult)
        assert np.array_equal(got.cpu().numpy().view(np.int8), want)


def test_producer_relu_and_row_major_scales(ctx):
    """The two options the int8 layer uses: negative results zeroed after the conversion (cpu_infer.cpp:520-524), and
    the scales laid out [row][head], the layout the cache append reads."""
    rng = np.random.default_rng(21)
    n, H, d = 37, 3, 128
    x = (rng.standard_normal((n, H * d)) * 1000).astype(np.int32)
    want_q, want_s = orc.rope_normalize_rows(capi.I8, x, H, scale_mult=0.5)
    xd = torch.from_numpy(x).cuda()
    q, s = ctx.rope_normalize_rows(xd, H, capi.I8, scale_mult=0.5, row_major_scale=True, relu=True)
    torch.cuda.synchronize()
    want_relu = want_q.view(np.int8).copy()
    want_relu[want_relu < 0] = 0
    assert np.array_equal(q.cpu().numpy().view(np.int8), want_relu)
    assert (want_relu == 0).mean() > 0.4 and (want_relu > 0).any()
    assert s.shape == (n, H) and np.array_equal(s.cpu().numpy(), want_s.T)
    with pytest.raises(capi.TsattnError):
        ctx.rope_normalize_rows(xd, H, capi.E4M3, relu=True)


def test_producer_fused_forms_equal_the_separate_calls(ctx):
    """One producer call standing in for several: the parts of a split-K product summed on the fly, rotation for the
    leading heads only, scales for a range of heads, the residual update before the normalisation.  Each against the
    oracle's separate steps, bit for bit."""
    rng = np.random.default_rng(33)
    n, H, d = 19, 2, 128
    hd4 = 4 * H * d     # a row holding the qk, qv, k and v heads
    parts = (rng.standard_normal((3, n, hd4)) * 3000).astype(np.int32)
    total = parts.sum(axis=0).astype(np.int32)
    pos = rng.integers(0, 50, n).astype(np.int32)
    rope = orc.fill_rope(d, 64)
    # the oracle's four separate calls on the summed product
    seg = lambda i: np.ascontiguousarray(total[:, i * H * d:(i + 1) * H * d])
    want = [orc.rope_normalize_rows(capi.I8, seg(0), H, pos=pos, rope=rope),
            orc.rope_normalize_rows(capi.I8, seg(1), H, pos=pos, rope=rope, scale_mult=0.37),
            orc.rope_normalize_rows(capi.I8, seg(2), H),
            orc.rope_normalize_rows(capi.I8, seg(3), H)]
    q, s = ctx.rope_normalize_rows(torch.from_numpy(parts).cuda(), 4 * H, capi.I8, pos=torch.from_numpy(pos).cuda(),
                                   rope=torch.from_numpy(rope).cuda(), scale_mult=0.37, row_major_scale=True,
                                   rope_heads=2 * H, scale_heads=(H, H))
    torch.cuda.synchronize()
    got = q.cpu().numpy()
    for i in range(4):
        assert np.array_equal(got[:, i * H * d:(i + 1) * H * d], want[i][0]), f"segment {i}"
    assert s.shape == (n, H) and np.array_equal(s.cpu().numpy(), want[1][1].T)

    # residual update, then normalisation of the updated state (AddScaled + NormalizeState)
    dim = 4 * d
    state = rng.standard_normal((n, dim)).astype(np.float32)
    delta = (rng.standard_normal((2, n, dim)) * 50000).astype(np.int32)
    scale = np.float32(3.1e-5)
    new_state = state + delta.sum(axis=0).astype(np.float32) * scale       # one rounding per operation, as in AddScaled
    want_q, _ = orc.rope_normalize_rows(capi.I8, new_state, dim // 128)
    st = torch.from_numpy(state).cuda()
    q, _ = ctx.rope_normalize_rows(torch.from_numpy(delta).cuda(), dim // 128, capi.I8, resid=st, resid_scale=float(scale))
    torch.cuda.synchronize()
    assert np.array_equal(st.cpu().numpy(), new_state)
    assert np.array_equal(q.cpu().numpy(), want_q)
