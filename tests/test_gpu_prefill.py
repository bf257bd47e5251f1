"""GPU: MFMA prefill through the C ABI against the prefill oracle (compute/gpt_cpu.cpp:391-441 with
8-bit operands).  int8 QK^T accumulators bit-exact; e4m3 accumulators within a few fp32 ulps of the
exact sum; outputs within max-abs 2e-2 / mean-abs 2e-3 on unit-variance outputs."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tests.common import assert_within_tolerance, make_qkv
from tscale_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=1, max_heads=16, max_head_dim=128)
    yield c
    c.close()


def run_gpu(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, slope, out_f16=False, want_acc=False, want_swl=False):
    n = q.shape[0]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    sc = lambda s: t(s) if isinstance(s, np.ndarray) else s
    dbg = None
    if want_acc:
        dbg = torch.zeros((H, n, n), dtype=torch.int32 if dtype == capi.I8 else torch.float32, device="cuda")
        dbg = dbg.view(H * n, n).unsqueeze(0)[0].view(H, n, n)
    swl = torch.zeros((H, n), dtype=torch.float32, device="cuda") if want_swl else None
    out = ctx.compute_val_lookup(dtype, H, t(q), t(k), t(v), sc(qs), sc(ks), sc(vs), t(st), t(fi), slope,
                                 out_f16=out_f16, sum_weight_log=swl,
                                 debug_qk_acc=None if dbg is None else dbg.view(H * n, n).view(H, n, n))
    torch.cuda.synchronize()
    res = [out.float().cpu().numpy()]
    if want_acc:
        res.append(dbg.cpu().numpy())
    if want_swl:
        res.append(swl.cpu().numpy())
    return res if len(res) > 1 else res[0]


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("window,slope", [(10 ** 6, 0.0), (64, 0.5), (0, 0.0), (1, 0.0), (256, 0.5)])
def test_prefill_parity_small(ctx, dtype, d, window, slope):
    H = 2
    seq_lens = [300, 1, 129, 70]  # ragged: sequence boundaries inside query tiles
    n = sum(seq_lens)
    q, qs, k, ks, v, vs = make_qkv(50 + d, n, H, d, dtype)
    st, fi = orc.make_spans(seq_lens, window)
    want, want_swl = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope, want_swl=True)
    out, acc, swl = run_gpu(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, slope, want_acc=True, want_swl=True)
    for h in range(H):
        for f in range(0, n, 7):
            if fi[f] < st[f]:
                continue
            ref = orc.qk_accum(dtype, q, k, h, d, f, 1, int(st[f]), int(fi[f] - st[f] + 1))[0]
            got = acc[h, f, st[f]:fi[f] + 1]
            if dtype == capi.I8:
                assert np.array_equal(got, ref), "int32 QK^T accumulators differ"
            else:
                # v_mfma_f32_32x32x64_f8f6f4 aligns the 64 products of a step to their largest exponent and
                # keeps fewer bits than fp32 there: the error is relative to the largest product a row pair
                # can hold (256*256 after absmax scaling), not to the sum.  2^-12 of that, measured ~2^-13.
                assert np.all(np.abs(got - ref) <= 2.0 ** -12 * 65536.0 + 2.0 ** -12 * np.abs(ref))
    assert_within_tolerance(out, want, "prefill")
    assert np.abs(swl - want_swl).max() < 1e-3
    empty = fi < st
    assert not out[empty].any()


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
def test_prefill_doc_boundaries_and_f16_out(ctx, dtype):
    H, d = 3, 128
    seq_lens = [513, 255]
    n = sum(seq_lens)
    flags = (np.random.default_rng(2).random(n) < 0.01).astype(np.uint8)
    q, qs, k, ks, v, vs = make_qkv(61, n, H, d, dtype)
    st, fi = orc.make_spans(seq_lens, 10 ** 6, flags)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0)
    out = run_gpu(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, 0.0, out_f16=True)
    assert_within_tolerance(out, want, "prefill f16 out")


def test_prefill_mask_probe_one_hot_values(ctx):
    """V = one-hot(to) makes the output equal to the weight vector: pins which keys each row sees."""
    H, d, n = 1, 128, 128
    rng = np.random.default_rng(3)
    q = rng.integers(-20, 21, (n, d)).astype(np.int8).view(np.uint8)
    k = rng.integers(-20, 21, (n, d)).astype(np.int8).view(np.uint8)
    v = np.eye(n, d, dtype=np.int8).view(np.uint8)  # key t has value e_t (t < 128)
    for window in (0, 1, 5, 64, 1000):
        st, fi = orc.make_spans([70, 58], window)
        out = run_gpu(ctx, capi.I8, H, q, 0.01, k, 0.02, v, 1.0, st, fi, 0.25)
        for f in range(n):
            seen = set(np.nonzero(out[f] > 0)[0].tolist())
            assert seen == set(range(st[f], fi[f] + 1)), (window, f)


def test_prefill_constant_scales_and_global_key_scale(ctx):
    H, d, n = 2, 128, 200
    rng = np.random.default_rng(4)
    q, k, v = (rng.integers(-127, 128, (n, H * d)).astype(np.int8).view(np.uint8) for _ in range(3))
    ks = (rng.random((H, n)).astype(np.float32) + 0.5) / 24
    VEC = 1.0 / 24
    st, fi = orc.make_spans([n], 64)
    want = orc.prefill_q8(orc.I8, q, k, v, H, VEC, ks * np.float32(0.37), VEC, st, fi, 0.5)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = ctx.compute_val_lookup(capi.I8, H, t(q), t(k), t(v), VEC, t(ks), VEC, t(st), t(fi), 0.5,
                                 k_global_scale=torch.tensor([0.37], device="cuda")).cpu().numpy()
    assert_within_tolerance(out, want, "constant scales")


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("d,window,slope,seq_lens", [
    (128, 10 ** 6, 0.0, [700, 324]),     # the common-tile loop, tiles on the diagonal, a sequence boundary inside a tile
    (128, 256, 0.5, [900]),              # ALiBi, both ends of the spans cut through tiles
    (64, 10 ** 6, 0.0, [513, 255]),
    (64, 64, 0.25, [400, 1, 130]),       # the short-range path of d = 64
])
def test_prefill_constant_query_scale(ctx, dtype, d, window, slope, seq_lens):
    """TScale's own model passes one number as the query scale (VEC_SCALE, gpt_att_fp8.cuh:137): the kernels that fold it
    into the staged key scales, per-row key and value scales as usual, f32 and f16 results, with sum_weight_log."""
    H, n = 3, sum(seq_lens)
    q, _, k, ks, v, vs = make_qkv(77, n, H, d, dtype)
    VEC = np.float32(1.0 / 48 if dtype == capi.I8 else 1.0 / 96)   # (logits of the usual size for these rows)
    st, fi = orc.make_spans(seq_lens, window)
    tt = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    for v_const in (False, True):   # ... and one number as the value scale too (cpu_infer.cpp:454): V widened as it is
        v_scale = float(np.float32(vs.mean())) if v_const else vs
        want, want_swl = orc.prefill_q8(dtype, q, k, v, H, float(VEC), ks, v_scale, st, fi, slope, want_swl=True)
        for f16 in (False, True):
            swl = torch.zeros((H, n), dtype=torch.float32, device="cuda")
            out = ctx.compute_val_lookup(dtype, H, tt(q), tt(k), tt(v), float(VEC), tt(ks), v_scale if v_const else tt(vs), tt(st), tt(fi), slope,
                                         out_f16=f16, sum_weight_log=swl)
            torch.cuda.synchronize()
            assert_within_tolerance(out.float().cpu().numpy(), want, f"constant query scale, constant value scale {v_const}, f16 out {f16}")
            assert np.abs(swl.cpu().numpy() - want_swl).max() < 1e-3


@pytest.mark.parametrize("dtype,B,S,H,d,window,slope", [
    (capi.I8, 1, 1024, 12, 64, 1024, 0.0),     # the CPU-reference configuration, full size
    (capi.E4M3, 2, 1024, 12, 64, 64, 0.5),     # 125M-style short-window layer, reduced batch
    (capi.E4M3, 2, 1024, 12, 64, 1024, 0.0),   # 125M-style wide layer, reduced batch
    (capi.E4M3, 1, 2048, 4, 128, 256, 0.5),    # 1.5B-style layers, reduced batch / heads / length
    (capi.E4M3, 1, 2048, 4, 128, 2048, 0.0),
])
def test_prefill_parity_benchmark_shapes(ctx, dtype, B, S, H, d, window, slope):
    n = B * S
    q, qs, k, ks, v, vs = make_qkv(1313, n, H, d, dtype)
    st, fi = orc.make_spans([S] * B, window)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope)
    out = run_gpu(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, slope)
    mx, mean = assert_within_tolerance(out, want, "benchmark shape")
    print(f"unit-variance error: max {mx:.2e} mean {mean:.2e}")


def test_prefill_full_size_properties(ctx):
    """1.5B-style shape at full size (B8 S4096 H16 d128 e4m3): V = ones of scale 1 gives
    out = 1 - 2^-sum_weight_log in every column, and row 0 of every sequence is zero."""
    B, S, H, d = 8, 4096, 16, 128
    n = B * S
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((n, H * d), device="cuda", generator=g)
    q, qs = ctx.quantize_rows(x, H, capi.E4M3)
    k, ks = ctx.quantize_rows(torch.randn((n, H * d), device="cuda", generator=g), H, capi.E4M3)
    v = torch.full((n, H * d), 0x38, dtype=torch.uint8, device="cuda")  # e4m3 1.0
    off = torch.arange(0, n + 1, S, dtype=torch.int32, device="cuda")
    st, fi = ctx.build_spans(off, n, S)
    swl = torch.zeros((H, n), device="cuda")
    out = ctx.compute_val_lookup(capi.E4M3, H, q, k, v, qs, ks, 1.0, st, fi, 0.0, sum_weight_log=swl)
    torch.cuda.synchronize()
    o = out.view(n, H, d)
    assert (o[::S] == 0).all()
    want = 1 - torch.exp2(-swl).t()
    assert (o - want[:, :, None]).abs().max().item() < 2e-3
    assert (o.max(dim=2).values - o.min(dim=2).values).max().item() < 1e-6


@pytest.mark.parametrize("dtype,d", [(capi.E4M3, 64), (capi.I8, 128)])
def test_prefill_launch_order_hint_never_changes_results(ctx, dtype, d):
    """causal_period only permutes the order in which query tiles are launched: with a usable value, a value the
    kernel cannot use (not a multiple of the tile, not dividing the batch) and a wrong one, the output is
    bit-identical to the one without a hint."""
    B, S, H = 8, 512, 4     # 32 query tiles x 4 heads = 128 workgroups: the reordering applies
    n = B * S
    q, qs, k, ks, v, vs = make_qkv(77, n, H, d, dtype)
    st, fi = orc.make_spans([S] * B, S)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    args = (dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), 0.0)
    base = ctx.compute_val_lookup(*args).cpu().numpy()
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0)
    assert_within_tolerance(base, want, "no hint")
    for period in (S, 2 * S, 256, 100, 384, n, 10 ** 9):
        got = ctx.compute_val_lookup(*args, causal_period=period).cpu().numpy()
        assert np.array_equal(got, base), f"causal_period={period}"


def test_prefill_logits_far_above_the_zero_vector(ctx):
    """Large query scales push logits tens of log2 units above the zero vector's 0: the reference maximum has to
    be raised several times, on interior tiles (the common-tile path's weight-sum check) and on the diagonal."""
    H, d = 2, 128
    seq_lens = [700, 330]
    n = sum(seq_lens)
    for dtype in (capi.E4M3, capi.I8):
        q, qs, k, ks, v, vs = make_qkv(31, n, H, d, dtype)
        for boost in (8.0, 40.0):
            qb = (qs * np.float32(boost)).astype(np.float32)
            st, fi = orc.make_spans(seq_lens, 10 ** 6)
            want, want_swl = orc.prefill_q8(dtype, q, k, v, H, qb, ks, vs, st, fi, 0.0, want_swl=True)
            out, swl = run_gpu(ctx, dtype, H, q, qb, k, ks, v, vs, st, fi, 0.0, want_swl=True)
            assert np.isfinite(out).all()
            assert want_swl.max() > 20.0 if boost > 10 else want_swl.max() > 4.0
            assert_within_tolerance(out, want, f"boost {boost}")
            assert np.abs(swl - want_swl).max() < 2e-3 * max(1.0, np.abs(want_swl).max() / 16)


@pytest.mark.parametrize("window,slope", [(10 ** 6, 0.0), (64, 0.5), (0, 0.0), (5, 0.2)])
def test_prefill_span_summary_gives_identical_results(ctx, window, slope):
    """With the per-128-row span summary (tsattn_build_span_tiles) the kernel skips its own span reduction; the
    summary equals a numpy reduction of the spans and the output is bit-identical to the run without it.  Ragged
    sequences, document starts, rows without keys, a last partial tile."""
    H, d, dtype = 2, 64, capi.E4M3
    seq_lens = [300, 1, 129, 70, 513]
    n = sum(seq_lens)
    rng = np.random.default_rng(3)
    flags = (rng.random(n) < 0.01).astype(np.uint8)
    q, qs, k, ks, v, vs = make_qkv(8, n, H, d, dtype)
    st, fi = orc.make_spans(seq_lens, window, flags)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    tiles = ctx.build_span_tiles(t(st), t(fi))
    got_tiles = tiles.cpu().numpy()
    n_tiles = (n + 127) // 128
    assert got_tiles.shape == (n_tiles, capi.SPAN_TILE_INTS)
    for i in range(n_tiles):
        a, b = st[i * 128:(i + 1) * 128], fi[i * 128:(i + 1) * 128]
        has = b >= a
        want_min = a[has].min() if has.any() else 0x7fffffff
        want_max = b[has].max() if has.any() else -1
        assert got_tiles[i, 0] == want_min and got_tiles[i, 1] == want_max
        for w in range(4):
            aw, bw = a[32 * w:32 * w + 32], b[32 * w:32 * w + 32]
            hw = bw >= aw
            e = got_tiles[i, 4 + 5 * w: 9 + 5 * w]
            if hw.any():
                assert e.tolist()[:4] == [aw[hw].min(), aw[hw].max(), bw[hw].min(), bw[hw].max()]
            else:
                assert e[0] > e[3]
            assert e[4] == int(len(aw) == 32 and hw.all())
    args = (dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), slope)
    base = ctx.compute_val_lookup(*args).cpu().numpy()
    with_tiles = ctx.compute_val_lookup(*args, span_tiles=tiles).cpu().numpy()
    assert np.array_equal(base, with_tiles)
    assert_within_tolerance(base, orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope), "span summary")


@pytest.mark.parametrize("dtype,d,H,n,window", [
    (capi.E4M3, 64, 3, 333, 10 ** 6),    # odd head count with d=64: no head pairing; 9 workgroups: no XCD remap
    (capi.I8, 64, 6, 1024, 100),         # 48 workgroups: remapped, heads paired
    (capi.I8, 128, 5, 257, 10 ** 6),     # one row in the last query tile
    (capi.E4M3, 128, 2, 640, 64),
])
def test_prefill_layout_variants(ctx, dtype, d, H, n, window):
    """Row pitches larger than a row, a scale pitch larger than the token count, f32 output into a padded buffer,
    a launch-order hint that does not apply, with and without the span summary: results as for packed arrays."""
    q, qs, k, ks, v, vs = make_qkv(3 * d + H, n, H, d, dtype)
    st, fi = orc.make_spans([n], window)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.25)
    pad = 48                      # bytes; keeps 16-byte alignment
    sp = n + 37                   # scale pitch
    def padded(a):
        t = torch.zeros((n, H * d + pad), dtype=torch.uint8, device="cuda")
        t[:, :H * d] = torch.from_numpy(a).cuda()
        return t[:, :H * d]       # a view whose stride(0) is the padded pitch
    def scale_plane(a):
        t = torch.zeros((H, sp), dtype=torch.float32, device="cuda")
        t[:, :n] = torch.from_numpy(a).cuda()
        return t[:, :n]
    out_buf = torch.full((n, H * d + 8), -7.0, dtype=torch.float32, device="cuda")
    out = out_buf[:, :H * d]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    for use_summary in (False, True):
        out_buf.fill_(-7.0)
        tiles = ctx.build_span_tiles(t(st), t(fi)) if use_summary else None
        a = capi.PrefillArgs()   # straight through the C ABI: the Python helper insists on contiguous scale planes
        qq, kk, vv = padded(q), padded(k), padded(v)
        sq, sk, sv = scale_plane(qs), scale_plane(ks), scale_plane(vs)
        a.dtype, a.out_dtype = dtype, capi.OUT_F32
        a.n_tokens, a.n_heads, a.head_dim = n, H, d
        a.q, a.k, a.v = qq.data_ptr(), kk.data_ptr(), vv.data_ptr()
        a.q_pitch = a.k_pitch = a.v_pitch = H * d + pad
        a.q_scale, a.k_scale, a.v_scale, a.scale_pitch = sq.data_ptr(), sk.data_ptr(), sv.data_ptr(), sp
        st_d, fi_d = t(st), t(fi)
        a.span_start, a.span_finish = st_d.data_ptr(), fi_d.data_ptr()
        a.span_tiles = None if tiles is None else tiles.data_ptr()
        a.alibi_slope = 0.25
        a.out, a.out_pitch = out.data_ptr(), (H * d + 8) * 4
        a.causal_period = 128
        import ctypes
        capi.check(ctx.lib.tsattn_prefill(ctx.handle, ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        assert_within_tolerance(out.cpu().numpy(), want, f"layout variant (summary {use_summary})")
        assert (out_buf[:, H * d:] == -7.0).all(), "wrote outside the rows"


@pytest.mark.parametrize("dtype,d,H,seq_lens,period", [
    (capi.E4M3, 64, 12, [100], 0),        # one query tile, six head pairs: every division of the launch mapping is by 1
    (capi.I8, 128, 5, [128], 0),          # one query tile, five heads
    (capi.I8, 128, 8, [1024], 1024),      # one sequence with a usable period: one unit per XCD, groups of one unit
    (capi.E4M3, 64, 16, [1024], 1024),    # the same with paired heads
    (capi.E4M3, 128, 8, [256, 256], 256), # two sequences, two query tiles each
])
def test_prefill_launch_mapping_with_unit_divisors(ctx, dtype, d, H, seq_lens, period):
    """Launch shapes in which the workgroup -> (head, query tile) mapping divides by 1 somewhere."""
    n = sum(seq_lens)
    q, qs, k, ks, v, vs = make_qkv(11 * H + d, n, H, d, dtype)
    st, fi = orc.make_spans(seq_lens, 10 ** 6)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = ctx.compute_val_lookup(dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), 0.0, causal_period=period)
    torch.cuda.synchronize()
    assert_within_tolerance(out.cpu().numpy(), want, "unit divisors")


@pytest.mark.parametrize("dtype,d,H,n,window", [
    (capi.E4M3, 64, 2, 333, 10 ** 6),    # long key range (tile loop): the last 64-key tile ends 51 rows past the end
    (capi.E4M3, 128, 2, 200, 10 ** 6),
    (capi.I8, 64, 2, 150, 64),           # short key range path
    (capi.I8, 128, 3, 333, 100),
])
def test_prefill_ignores_what_lies_past_the_last_token(ctx, dtype, d, H, n, window):
    """Key tiles are 64 rows, so the last one usually reaches past n_tokens.  Whatever lies there (here: NaN scales
    and 0xff bytes, the e4m3 NaN) must not reach the output: 0 * NaN is NaN, so a masked weight does not hide it."""
    q, qs, k, ks, v, vs = make_qkv(5 * d + n, n, H, d, dtype)
    st, fi = orc.make_spans([n], window)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.125)
    extra = 130
    def rows(a):
        t = torch.full((n + extra, H * d), 0xff, dtype=torch.uint8, device="cuda")
        t[:n] = torch.from_numpy(a).cuda()
        return t
    def scales(a):
        t = torch.full((H, n + extra), float("nan"), dtype=torch.float32, device="cuda")
        t[:, :n] = torch.from_numpy(a).cuda()
        return t
    import ctypes
    qq, kk, vv = rows(q), rows(k), rows(v)
    sq, sk, sv = scales(qs), scales(ks), scales(vs)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    st_d, fi_d = t(st), t(fi)
    out = torch.zeros((n, H * d), dtype=torch.float32, device="cuda")
    a = capi.PrefillArgs()
    a.dtype, a.out_dtype = dtype, capi.OUT_F32
    a.n_tokens, a.n_heads, a.head_dim = n, H, d
    a.q, a.k, a.v = qq.data_ptr(), kk.data_ptr(), vv.data_ptr()
    a.q_pitch = a.k_pitch = a.v_pitch = H * d
    a.q_scale, a.k_scale, a.v_scale, a.scale_pitch = sq.data_ptr(), sk.data_ptr(), sv.data_ptr(), n + extra
    a.span_start, a.span_finish = st_d.data_ptr(), fi_d.data_ptr()
    a.alibi_slope = 0.125
    a.out, a.out_pitch = out.data_ptr(), H * d * 4
    capi.check(ctx.lib.tsattn_prefill(ctx.handle, ctypes.byref(a), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.isfinite(got).all(), "rows past the last token reached the output"
    assert_within_tolerance(got, want, "rows past the end")


@pytest.mark.parametrize("seed", range(10))
def test_prefill_randomised_shapes(ctx, seed):
    """Seeded random launch shapes: head counts, ragged sequence lists (some of one token, some crossing many query
    tiles), windows from 0 to beyond the longest sequence, document starts, slopes, period hints that apply, do not apply
    or are wrong, with and without the span summary; always against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    dtype = [capi.I8, capi.E4M3][seed % 2]
    d = [64, 128][(seed // 2) % 2]
    H = int(rng.choice([1, 2, 3, 5, 8, 12, 16]))
    n_seq = int(rng.integers(1, 7))
    seq_lens = [int(x) for x in rng.choice([1, 2, 63, 64, 65, 127, 128, 129, 200, 333, 512, 700], n_seq)]
    if seed % 3 == 0:
        seq_lens = [int(rng.choice([128, 256, 384]))] * n_seq      # equal lengths: the period hint can apply
    n = sum(seq_lens)
    window = int(rng.choice([0, 1, 2, 31, 64, 100, 256, 10 ** 6]))
    slope = float(rng.choice([0.0, 0.0, 0.25, 0.5]))
    flags = (rng.random(n) < 0.01).astype(np.uint8) if seed % 2 else None
    q, qs, k, ks, v, vs = make_qkv(900 + seed, n, H, d, dtype)
    st, fi = orc.make_spans(seq_lens, window, flags)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    args = (dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), slope)
    tiles = ctx.build_span_tiles(t(st), t(fi))
    period = int(rng.choice([0, seq_lens[0], 128, 2 * seq_lens[0], 96]))
    outs = [ctx.compute_val_lookup(*args).cpu().numpy(),
            ctx.compute_val_lookup(*args, span_tiles=tiles, causal_period=period).cpu().numpy()]
    what = f"seed {seed}: dtype {dtype} d {d} H {H} seqs {seq_lens} window {window} slope {slope} period {period}"
    assert np.array_equal(outs[0], outs[1]), what
    assert_within_tolerance(outs[0], want, what)
    assert not outs[0][fi < st].any(), what


@pytest.mark.parametrize("d,H,seq_lens,window,slope,rep", [
    (128, 3, [300, 1, 129, 70], 10 ** 6, 0.0, 4),
    (128, 2, [257], 64, 0.5, 3),
    (64, 5, [40, 200, 333], 10 ** 6, 0.0, 4),
    (64, 2, [128, 128], 1, 0.25, 1),
    (64, 1, [100], 0, 0.0, 2),
])
def test_prefill_fused_kv_product_equals_the_separate_call(ctx, d, H, seq_lens, window, slope, rep):
    """KVProduct as the prefill kernel's last step: the same bytes as tsattn_kv_product on the f32 result of the same
    launch (which the oracle's KVProduct of that result confirms), with and without the result itself written, with
    the K rows and the output inside wider rows, and nothing written outside the output's columns."""
    n = sum(seq_lens)
    q, qs, k, ks, v, vs = make_qkv(70 + d + rep, n, H, d, capi.I8)
    st, fi = orc.make_spans(seq_lens, window)
    rng = np.random.default_rng(5 + rep)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    wide = t(rng.integers(-127, 128, (n, H * d + 64), dtype=np.int8).view(np.uint8))
    kk = wide[:, 32:32 + H * d]   # 4-byte aligned rows of a wider array
    mult = 0.37
    args = (capi.I8, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), slope)
    room = torch.full((n, H * d * rep + 48), 0x5a, dtype=torch.uint8, device="cuda")
    kv_out = room[:, 16:16 + H * d * rep]
    out = ctx.compute_val_lookup(*args, kv_product=(kk, kv_out, rep, mult))
    plain = ctx.compute_val_lookup(*args)
    assert torch.equal(out, plain), "the result itself changes with the fused consumer"
    separate = ctx.kv_product(kk.contiguous(), plain, H, rep, mult)
    assert torch.equal(kv_out, separate), "fused KVProduct differs from the separate call"
    want = orc.kv_product(kk.cpu().numpy(), plain.cpu().numpy(), H, rep, mult)
    assert np.array_equal(kv_out.cpu().numpy().view(np.int8), want)
    assert (room[:, :16] == 0x5a).all() and (room[:, 16 + H * d * rep:] == 0x5a).all()
    # without the result, with the span summary and a period hint
    kv2 = torch.zeros((n, H * d * rep), dtype=torch.uint8, device="cuda")
    tiles = ctx.build_span_tiles(t(st), t(fi))
    none = ctx.compute_val_lookup(*args, kv_product=(kk, kv2, rep, mult), want_out=False, span_tiles=tiles, causal_period=seq_lens[0])
    assert none is None and torch.equal(kv2, separate)


def test_prefill_fused_kv_product_argument_checks(ctx):
    n, H, d = 64, 1, 64
    q, qs, k, ks, v, vs = make_qkv(3, n, H, d, capi.E4M3)
    st, fi = orc.make_spans([n], 10 ** 6)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    kk = torch.zeros((n, H * d), dtype=torch.uint8, device="cuda")
    kv = torch.zeros((n, H * d * 4), dtype=torch.uint8, device="cuda")
    with pytest.raises(capi.TsattnError):      # e4m3 attention: no fused consumer
        ctx.compute_val_lookup(capi.E4M3, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), 0.0, kv_product=(kk, kv, 4, 1.0))
    q, qs, k, ks, v, vs = make_qkv(3, n, H, d, capi.I8)
    args = (capi.I8, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), 0.0)
    with pytest.raises(capi.TsattnError):      # f16 result
        ctx.compute_val_lookup(*args, out_f16=True, kv_product=(kk, kv, 4, 1.0))
    with pytest.raises(capi.TsattnError):      # rep out of range
        ctx.compute_val_lookup(*args, kv_product=(kk, kv, 5, 1.0))
    with pytest.raises(capi.TsattnError):      # output rows too short
        ctx.compute_val_lookup(*args, kv_product=(kk, kv[:, :H * d * 2].contiguous(), 4, 1.0))


@pytest.mark.parametrize("seed", range(8))
def test_prefill_arbitrary_spans(ctx, seed):
    """Spans that no window mask makes: every row its own random [start, finish] anywhere in the batch (before it, after
    it, across it), a fifth of the rows without keys, short and long ones mixed inside every 32-row group, so that the
    tile classes a wave sees (not needed, cut at either end or both, fully inside) come in every order.  The reference
    computes whatever TAttentionInfo lists (gpt/compute/gpt_cpu.cpp:391-441); so must the kernel, with and without the
    span summary."""
    rng = np.random.default_rng(7000 + seed)
    dtype = [capi.I8, capi.E4M3][seed % 2]
    d = [128, 64][(seed // 2) % 2]
    H = int(rng.choice([1, 2, 4]))
    n = int(rng.choice([97, 256, 300, 515, 777]))
    slope = float(rng.choice([0.0, 0.25]))
    st = rng.integers(0, n, n).astype(np.int32)
    length = rng.choice([1, 2, 17, 40, 64, 65, 130, 300, n], n)
    fi = np.minimum(st + length - 1, n - 1).astype(np.int32)
    empty = rng.random(n) < 0.2
    fi[empty] = st[empty] - 1
    if seed >= 4:   # whole 32-row groups without keys, and one group that sees everything
        fi[32:64] = st[32:64] - 1
        st[64:96], fi[64:96] = 0, n - 1
    q, qs, k, ks, v, vs = make_qkv(7100 + seed, n, H, d, dtype)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    args = (dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), t(st), t(fi), slope)
    outs = [ctx.compute_val_lookup(*args).cpu().numpy(),
            ctx.compute_val_lookup(*args, span_tiles=ctx.build_span_tiles(t(st), t(fi))).cpu().numpy()]
    what = f"seed {seed}: dtype {dtype} d {d} H {H} n {n} slope {slope}"
    assert np.array_equal(outs[0], outs[1]), what
    assert_within_tolerance(outs[0], want, what)
    assert not outs[0][fi < st].any(), what


@pytest.mark.parametrize("dtype,d,H,n,window,slope", [
    (capi.E4M3, 128, 1, 700, 10 ** 6, 0.0),   # common-tile path, 11 key tiles
    (capi.I8, 64, 2, 600, 300, 0.25),         # windowed: the key range of the later workgroups starts far into the arrays
    (capi.I8, 64, 2, 150, 10 ** 6, 0.0),      # d = 64, at most 192 keys: the path without a tile loop
])
def test_prefill_largest_key_row_pitch(ctx, dtype, d, H, n, window, slope):
    """K and V rows TSATTN_PREFILL_MAX_KV_PITCH (8 MiB) apart: a 64-key tile spans 512 MiB, so the kernel's running
    32-bit offsets pass 1 GiB every second tile and are folded back into the 64-bit base again and again; the arrays
    end beyond 4 GiB, more than one buffer descriptor covers.  Results as for packed arrays; one byte more of pitch is
    refused."""
    import ctypes
    pitch = 8 << 20
    q, qs, k, ks, v, vs = make_qkv(7 * d + n, n, H, d, dtype)
    st, fi = orc.make_spans([n], window)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, slope)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    def spread(a):   # only the rows' first H*d bytes are ever written or read
        buf = torch.empty((n, pitch), dtype=torch.uint8, device="cuda")
        buf[:, :H * d] = t(a)
        return buf
    kk, vv = spread(k), spread(v)
    qq, sq, sk, sv, st_d, fi_d = t(q), t(qs), t(ks), t(vs), t(st), t(fi)
    out = torch.empty((n, H * d), dtype=torch.float32, device="cuda")
    a = capi.PrefillArgs()
    a.dtype, a.out_dtype = dtype, capi.OUT_F32
    a.n_tokens, a.n_heads, a.head_dim = n, H, d
    a.q, a.k, a.v = qq.data_ptr(), kk.data_ptr(), vv.data_ptr()
    a.q_pitch, a.k_pitch, a.v_pitch = H * d, pitch, pitch
    a.q_scale, a.k_scale, a.v_scale, a.scale_pitch = sq.data_ptr(), sk.data_ptr(), sv.data_ptr(), n
    a.span_start, a.span_finish = st_d.data_ptr(), fi_d.data_ptr()
    a.alibi_slope = slope
    a.out, a.out_pitch = out.data_ptr(), H * d * 4
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    capi.check(ctx.lib.tsattn_prefill(ctx.handle, ctypes.byref(a), stream))
    torch.cuda.synchronize()
    assert_within_tolerance(out.cpu().numpy(), want, "rows 8 MiB apart")
    a.k_pitch = pitch + 16
    with pytest.raises(capi.TsattnError):
        capi.check(ctx.lib.tsattn_prefill(ctx.handle, ctypes.byref(a), stream))


@pytest.mark.parametrize("dtype,d,H,n,max_spans,slope,out_f16", [
    (capi.I8, 128, 2, 300, 3, 0.0, False),
    (capi.E4M3, 64, 3, 257, 2, 0.25, True),
    (capi.I8, 64, 1, 200, 5, 0.5, False),
])
def test_prefill_rows_with_several_spans(ctx, dtype, d, H, n, max_spans, slope, out_f16):
    """Rows with any number of spans (TAttentionInfo, gpt/att/att.h:24-47): one tsattn_prefill launch that walks the parts
    (n_span_parts), and the fallback of one launch per span of the rows plus tsattn_merge_lookups, both against the
    oracle's loop over a row's spans inside one softmax (gpt_cpu.cpp:405-436) on the dequantised operands, and against
    each other within 1e-6 of the output's scale.  Spans overlap (a key in two spans counts twice), some rows have none."""
    from tests.test_oracle_attention import random_span_lists
    rng = np.random.default_rng(100 * d + n)
    q, qs, k, ks, v, vs = make_qkv(5 * d + n, n, H, d, dtype)
    ptr, spans = random_span_lists(rng, n, max_spans)
    tab = orc.e4m3_table()
    def deq(x, s):
        xf = x.view(np.int8).astype(np.float32) if dtype == capi.I8 else tab[x]
        return (xf.reshape(n, H, d) * s.T[:, :, None]).reshape(n, H * d)
    want, sw, mx = orc.prefill_f32(deq(q, qs), deq(k, ks), deq(v, vs), H, ptr, spans, slope)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    swl = torch.zeros((H, n), dtype=torch.float32, device="cuda")
    out = ctx.compute_val_lookup_multi(dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), ptr, spans, slope,
                                       out_f16=out_f16, sum_weight_log=swl)
    torch.cuda.synchronize()
    assert out.dtype == (torch.float16 if out_f16 else torch.float32)
    assert_within_tolerance(out.float().cpu().numpy(), want, "several spans per row")
    none = ptr[1:] == ptr[:-1]
    assert none.any() and not out[torch.from_numpy(none).cuda()].any()
    # sum_weight_log = max logit + log2(sum of the shifted weights, zero vector included)
    assert np.abs(swl.cpu().numpy() - (mx + np.log2(sw))).max() < 2e-3
    # the fallback: a launch per part and the merge
    swl2 = torch.zeros((H, n), dtype=torch.float32, device="cuda")
    out2 = ctx.compute_val_lookup_multi(dtype, H, t(q), t(k), t(v), t(qs), t(ks), t(vs), ptr, spans, slope,
                                        out_f16=out_f16, sum_weight_log=swl2, merge=True)
    torch.cuda.synchronize()
    assert_within_tolerance(out2.float().cpu().numpy(), want, "several spans per row, merged launches")
    if not out_f16:
        # The same sums in another order (the merge adds the parts' f32 results; the single launch keeps one accumulator):
        # equal to f32 rounding while no logit is far above the zero vector's.  Where one is (a span of keys behind the
        # row under a slope), the two raise the reference maximum at different moments and round their f16 weights against
        # different references.
        diff = (out - out2).abs().max().item()
        print(f"single launch vs merged launches: max abs difference {diff:.2e} (largest logit {mx.max():.1f})")
        assert diff <= (2e-6 if mx.max() <= 8.0 else 1e-3) * max(1.0, float(np.abs(want).max()))
    assert (swl - swl2).abs().max().item() < 2e-3


def test_merge_lookups_argument_checks(ctx):
    import ctypes
    parts = torch.zeros((2, 8, 64), dtype=torch.float32, device="cuda")
    swl = torch.zeros((2, 1, 8), dtype=torch.float32, device="cuda")
    assert not ctx.merge_lookups(parts, swl).any()        # two empty parts: an empty result
    with pytest.raises(capi.TsattnError):                  # parts that overlap
        ctx.merge_lookups(parts.as_strided((2, 8, 64), (64, 64, 1)), swl)
    a = capi.MergeArgs()
    a.n_parts, a.n_tokens, a.n_heads, a.head_dim = 0, 8, 1, 64
    with pytest.raises(capi.TsattnError):                  # no parts
        capi.check(ctx.lib.tsattn_merge_lookups(ctx.handle, ctypes.byref(a), None))
