"""GPU: the long-span prefill kernel (workspace + span_len_hint in tsattn_prefill_args) through the C ABI against the
prefill oracle (compute/gpt_cpu.cpp:391-441 with 8-bit operands), to the same bar as the standard kernel: outputs within
max-abs 2e-2 / mean-abs 2e-3 on unit-variance outputs, sum_weight_log within 1e-3, rows without keys exact zeros."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tests.common import assert_within_tolerance, make_qkv
from tscale_amd import capi

pytestmark = pytest.mark.gpu
D = 128


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=1, max_heads=16, max_head_dim=128)
    yield c
    c.close()


def t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_long(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, out_f16=False, want_swl=False, hint=8192, **kw):
    sc = lambda s: t(s) if isinstance(s, np.ndarray) else s
    n = q.shape[0]
    swl = torch.zeros((H, n), dtype=torch.float32, device="cuda") if want_swl else None
    out = ctx.compute_val_lookup(dtype, H, t(q), t(k), t(v), sc(qs), sc(ks), sc(vs), t(st), t(fi), 0.0, out_f16=out_f16,
                                 sum_weight_log=swl, span_len_hint=hint, **kw)
    torch.cuda.synchronize()
    out = out.float().cpu().numpy()
    return (out, swl.cpu().numpy()) if want_swl else out


def test_workspace_size_and_selection(ctx):
    """The workspace the header promises is what the wrapper allocates; without a hint the call needs none."""
    lib = capi.load()
    assert lib.tsattn_prefill_workspace_bytes(1000, 4, 64) == 0
    need = lib.tsattn_prefill_workspace_bytes(1000, 4, 128)
    assert need >= 4 * 128 * 1000 * 2
    q, qs, k, ks, v, vs = make_qkv(3, 300, 2, D, capi.E4M3)
    st, fi = orc.make_spans([300], 10 ** 6)
    a = run_long(ctx, capi.E4M3, 2, q, qs, k, ks, v, vs, st, fi, hint=0)
    assert ctx._workspace is None
    b = run_long(ctx, capi.E4M3, 2, q, qs, k, ks, v, vs, st, fi, hint=300)   # below the threshold: the standard kernel
    assert np.array_equal(a, b)
    c = run_long(ctx, capi.E4M3, 2, q, qs, k, ks, v, vs, st, fi, hint=8192)
    assert ctx._workspace is not None and np.abs(c - a).max() < 5e-3


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("seq_lens,H,window,doc_p", [
    ([300, 1, 129, 70], 2, 10 ** 6, None),   # ragged: sequence boundaries inside query tiles, a one-token sequence
    ([1024], 2, 10 ** 6, None),
    ([700, 324], 3, 10 ** 6, None),
    ([513, 255], 3, 10 ** 6, 0.01),          # document starts cut spans short
    ([900], 2, 200, None),                   # a window: both ends of the spans cut through tiles
    ([640], 1, 0, None),                     # window 0: every row sees itself only
    ([130], 1, 1, None),
])
def test_long_parity(ctx, dtype, seq_lens, H, window, doc_p):
    n = sum(seq_lens)
    q, qs, k, ks, v, vs = make_qkv(1313, n, H, D, dtype)
    flags = None if doc_p is None else (np.random.default_rng(2).random(n) < doc_p).astype(np.uint8)
    st, fi = orc.make_spans(seq_lens, window, flags) if flags is not None else orc.make_spans(seq_lens, window)
    want, want_swl = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0, want_swl=True)
    for f16 in (False, True):
        out, swl = run_long(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, out_f16=f16, want_swl=True)
        assert_within_tolerance(out, want, f"long-span prefill, f16 out {f16}")
        assert np.abs(swl - want_swl).max() < 1e-3
        assert not out[fi < st].any()


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
def test_long_parity_benchmark_shape_reduced(ctx, dtype):
    """The 1.5B-style full-window layer at reduced batch and heads, with the launch-order hint and the span summary."""
    S, H = 2048, 4
    q, qs, k, ks, v, vs = make_qkv(1313, S, H, D, dtype)
    st, fi = orc.make_spans([S], S)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0)
    tiles = ctx.build_span_tiles(t(st), t(fi))
    out = run_long(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, out_f16=True, causal_period=S, span_tiles=tiles)
    mx, mean = assert_within_tolerance(out, want, "long-span prefill, benchmark shape")
    print(f"unit-variance error: max {mx:.2e} mean {mean:.2e}")
    plain = run_long(ctx, dtype, H, q, qs, k, ks, v, vs, st, fi, out_f16=True)
    assert np.array_equal(out, plain), "hints change only the order of the work"


@pytest.mark.parametrize("mult", [6.0, 8.0, 40.0])
def test_long_logits_far_above_the_zero_vector(ctx, mult):
    """Weights that overflow f16 against the zero vector's logit: the workgroup repeats its rows on the path that
    tracks the maximum (rows next to them in the same workgroup included)."""
    dtype, H, n = capi.I8, 2, 700
    q, qs, k, ks, v, vs = make_qkv(7, n, H, D, dtype)
    st, fi = orc.make_spans([n], 10 ** 6)
    want, want_swl = orc.prefill_q8(dtype, q, k, v, H, qs * np.float32(mult), ks, vs, st, fi, 0.0, want_swl=True)
    assert want_swl.max() > 16
    out, swl = run_long(ctx, dtype, H, q, qs * np.float32(mult), k, ks, v, vs, st, fi, want_swl=True)
    assert np.isfinite(out).all()
    assert_within_tolerance(out, want, "logits far above the zero vector's")
    assert np.abs(swl - want_swl).max() < 2e-3


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
@pytest.mark.parametrize("ks_plane,gscale", [(True, None), (True, 0.37), (False, None), (False, 0.37)])
def test_long_constant_query_scale(ctx, dtype, ks_plane, gscale):
    """TScale's own model: q and v scales are the constant VEC_SCALE (cpu_infer.cpp:16), the key scales a plane or a
    constant, times the QV matrix scale (gpt_cuda.cu:476)."""
    H, n = 2, 600
    VEC = np.float32(1.0 / 24)
    q, _, k, ks, v, _ = make_qkv(11, n, H, D, dtype)
    scale = ks / ks.mean() * (VEC if dtype == capi.I8 else VEC / 4) if ks_plane else np.float32(VEC if dtype == capi.I8 else VEC / 4)
    st, fi = orc.make_spans([n], 10 ** 6)
    g = np.float32(1.0 if gscale is None else gscale)
    want = orc.prefill_q8(dtype, q, k, v, H, float(VEC), scale * g, float(VEC), st, fi, 0.0)
    kw = {} if gscale is None else {"k_global_scale": torch.tensor([gscale], device="cuda")}
    out = run_long(ctx, dtype, H, q, float(VEC), k, scale if ks_plane else float(scale), v, float(VEC), st, fi, **kw)
    assert_within_tolerance(out, want, "constant query scale")


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
def test_long_row_query_scales_with_constant_key_scale(ctx, dtype):
    """Query scales per row, one number as the key scale and the device scalar on top of it (the general kernel, whose
    key scales are then a constant in LDS and whose query scales carry the scalar)."""
    H, n = 2, 450
    q, qs, k, ks, v, vs = make_qkv(31, n, H, D, dtype)
    kc = float(np.float32(ks.mean()))
    st, fi = orc.make_spans([n], 10 ** 6)
    want = orc.prefill_q8(dtype, q, k, v, H, qs, kc * np.float32(0.6), vs, st, fi, 0.0)
    out = run_long(ctx, dtype, H, q, qs, k, kc, v, vs, st, fi, k_global_scale=torch.tensor([0.6], device="cuda"))
    assert_within_tolerance(out, want, "row query scales, constant key scale, global scale")


@pytest.mark.parametrize("dtype", [capi.I8, capi.E4M3])
def test_long_padded_rows_and_planes(ctx, dtype):
    """Q, K, V and the output as column slices of wider arrays (row pitches larger than a row, each different), scale
    planes with a pitch larger than the token count, one head: the kernel's row addresses come from the pitches."""
    H, n = 1, 333
    q, qs, k, ks, v, vs = make_qkv(21, n, H, D, dtype)
    st, fi = orc.make_spans([200, 133], 10 ** 6)
    want, want_swl = orc.prefill_q8(dtype, q, k, v, H, qs, ks, vs, st, fi, 0.0, want_swl=True)
    def wide(a, extra, fill):
        w = torch.full((a.shape[0], a.shape[1] + extra), fill, dtype=torch.uint8, device="cuda")
        w[:, :a.shape[1]] = t(a)
        return w[:, :a.shape[1]]
    planes = torch.full((4, H, n + 40), 7.0, dtype=torch.float32, device="cuda")   # q, k, v scales and sum_weight_log
    for i, sc in enumerate((qs, ks, vs)):
        planes[i, :, :n] = t(sc)
    out_w = torch.full((n, H * D + 48), -5.0, dtype=torch.float32, device="cuda")
    out = ctx.compute_val_lookup(dtype, H, wide(q, 16, 0x7F), wide(k, 64, 0x7F), wide(v, 32, 0x7F), planes[0, :, :n], planes[1, :, :n], planes[2, :, :n],
                                 t(st), t(fi), 0.0, out=out_w[:, :H * D], sum_weight_log=planes[3, :, :n], span_len_hint=8192)
    torch.cuda.synchronize()
    assert_within_tolerance(out.cpu().numpy(), want, "padded rows")
    assert np.abs(planes[3, :, :n].cpu().numpy() - want_swl).max() < 1e-3
    assert bool((out_w[:, H * D:] == -5.0).all()) and bool((planes[3, :, n:] == 7.0).all()), "nothing written outside the rows"


def test_long_full_size_properties(ctx):
    """1.5B-style shape at full size (B8 S4096 H16 d128 e4m3): V = ones of scale 1 gives out = 1 - 2^-sum_weight_log in
    every column, row 0 of every sequence is zero, and the result equals the standard kernel's within the f16 rounding
    of the weights."""
    B, S, H = 8, 4096, 16
    n = B * S
    g = torch.Generator(device="cuda").manual_seed(1313)
    q, qs = ctx.quantize_rows(torch.randn((n, H * D), device="cuda", generator=g), H, capi.E4M3)
    k, ks = ctx.quantize_rows(torch.randn((n, H * D), device="cuda", generator=g), H, capi.E4M3)
    v = torch.full((n, H * D), 0x38, dtype=torch.uint8, device="cuda")  # e4m3 1.0
    st = (torch.arange(n, device="cuda", dtype=torch.int32) // S) * S
    fi = torch.arange(n, device="cuda", dtype=torch.int32) - 1
    swl = torch.zeros((H, n), dtype=torch.float32, device="cuda")
    out = ctx.compute_val_lookup(capi.E4M3, H, q, k, v, qs, ks, 1.0, st, fi, 0.0, sum_weight_log=swl, causal_period=S, span_len_hint=2 * S)
    base = ctx.compute_val_lookup(capi.E4M3, H, q, k, v, qs, ks, 1.0, st, fi, 0.0, causal_period=S)
    torch.cuda.synchronize()
    want = (1.0 - torch.exp2(-swl)).t()                     # [n, H]
    got = out.view(n, H, D)
    assert (got - want[:, :, None]).abs().max().item() < 2e-3
    assert not out[::S].any()
    assert (out - base).abs().max().item() < 2e-3
