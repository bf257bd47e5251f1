"""GPU: int8 matrix product through the C ABI against the oracle's MulForward / AddScaled
(gpt/train/cpu_infer.cpp:294-316).  Integer sums bit-exact; the scaled forms bit-exact too (one multiply and one
add per element, rounded as in the reference's two statements)."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc
from tscale_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=1, max_heads=16, max_head_dim=128)
    yield c
    c.close()


def rand_i8(rng, shape):
    return rng.integers(-127, 128, shape).astype(np.int8)


dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("m,n,k", [
    (1, 32, 64), (32, 2048, 2048), (31, 100, 192), (33, 33, 64), (64, 40, 1024), (128, 96, 320),     # few rows
    (129, 128, 64), (300, 257, 192), (1000, 130, 2048), (256, 256, 4096), (131, 1, 128),             # many rows
    (8192, 4096, 128), (8000, 4100, 64), (8000, 4100, 384), (4096, 8192, 1024),                      # the largest output tiles
])
def test_matmul_int32_bit_exact(ctx, m, n, k):
    rng = np.random.default_rng(m + 7 * n + k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    want = orc.matmul_i8(a, w)
    got = ctx.matmul_i8(dev(a.view(np.uint8)), dev(w.view(np.uint8)))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("m", [32, 200])
def test_matmul_extremes(ctx, m):
    k, n = 8192, 64
    a = np.full((m, k), 127, dtype=np.int8); a[1::2] = -127
    w = np.full((n, k), 127, dtype=np.int8); w[3] = -127
    got = ctx.matmul_i8(dev(a.view(np.uint8)), dev(w.view(np.uint8))).cpu().numpy()
    assert np.array_equal(got, orc.matmul_i8(a, w))
    assert got[0, 0] == 127 * 127 * k and got[1, 0] == -127 * 127 * k and got[0, 3] == -127 * 127 * k


@pytest.mark.parametrize("m,n,k", [(32, 256, 512), (160, 192, 256), (4100, 8190, 128)])
def test_matmul_scaled_forms_and_pitches(ctx, m, n, k):
    """f32 output, AddScaled into a state with a padded pitch, operands with padded pitches; nothing outside the
    [m, n] block is written."""
    rng = np.random.default_rng(k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    scale = 0.0371
    ap = torch.zeros((m, k + 48), dtype=torch.uint8, device="cuda"); ap[:, :k] = dev(a.view(np.uint8))
    wp = torch.full((n, k + 16), 77, dtype=torch.uint8, device="cuda"); wp[:, :k] = dev(w.view(np.uint8))
    f = ctx.matmul_i8(ap[:, :k], wp[:, :k], mode=capi.MM_F32, scale=scale).cpu().numpy()
    assert np.array_equal(f, orc.matmul_i8(a, w, mode=1, scale=scale))
    state = rng.standard_normal((m, n)).astype(np.float32)
    buf = torch.full((m, n + 5), -3.0, dtype=torch.float32, device="cuda")
    buf[:, :n] = dev(state)
    ctx.matmul_i8(ap[:, :k], wp[:, :k], mode=capi.MM_ADD_SCALED, scale=scale, out=buf[:, :n])
    torch.cuda.synchronize()
    assert np.array_equal(buf[:, :n].cpu().numpy(), orc.matmul_i8(a, w, mode=2, scale=scale, out=state))
    assert (buf[:, n:] == -3.0).all()


def test_matmul_argument_checks(ctx):
    a = torch.zeros((4, 96), dtype=torch.uint8, device="cuda")
    w = torch.zeros((4, 96), dtype=torch.uint8, device="cuda")
    with pytest.raises(capi.TsattnError):
        ctx.matmul_i8(a, w)          # k not a multiple of 64
    # empty products are accepted and touch nothing
    e = ctx.matmul_i8(torch.zeros((0, 64), dtype=torch.uint8, device="cuda"), torch.zeros((4, 64), dtype=torch.uint8, device="cuda"))
    assert e.shape == (0, 4)


@pytest.mark.parametrize("m,n,k,mode", [(32, 2048, 8192, capi.MM_ADD_SCALED), (1, 96, 1024, capi.MM_I32), (128, 2048, 2048, capi.MM_F32),
                                        (33, 1000, 4096, capi.MM_ADD_SCALED)])
def test_matmul_split_k_with_a_workspace_gives_the_same_bits(ctx, m, n, k, mode):
    """Few rows: with room for partial sums K is split over more workgroups; sums are integers, so nothing changes."""
    rng = np.random.default_rng(n)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    state = rng.standard_normal((m, n)).astype(np.float32)
    want = orc.matmul_i8(a, w, mode=mode, scale=0.002, out=state if mode == capi.MM_ADD_SCALED else None)
    for ws_bytes in (0, 2 * 4 * m * n, 16 * 4 * m * n + 64):
        ws = torch.full((ws_bytes,), 0xAB, dtype=torch.uint8, device="cuda") if ws_bytes else None
        out = dev(state) if mode == capi.MM_ADD_SCALED else None
        got = ctx.matmul_i8(dev(a.view(np.uint8)), dev(w.view(np.uint8)), mode=mode, scale=0.002, out=out, workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want), f"workspace {ws_bytes} bytes"


@pytest.mark.parametrize("m,n,k", [(32, 2048, 8192), (5, 96, 128), (300, 130, 256)])
def test_matmul_planes_sum_to_the_product(ctx, m, n, k):
    """TSATTN_MM_I32_PLANES: the parts of a split-K product left as int32 planes for a consumer that adds them up."""
    rng = np.random.default_rng(m * n)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    planes = ctx.matmul_i8(dev(a.view(np.uint8)), dev(w.view(np.uint8)), mode=capi.MM_I32_PLANES)
    torch.cuda.synchronize()
    assert 1 <= planes.shape[0] <= 16 and planes.shape[1:] == (m, n)
    if (m, n, k) == (32, 2048, 8192):
        assert planes.shape[0] > 1, "this shape is meant to split K"
    assert np.array_equal(planes.sum(dim=0, dtype=torch.int32).cpu().numpy(), orc.matmul_i8(a, w))


@pytest.mark.parametrize("m,n,k,d,variant", [
    (4096, 8192, 256, 128, "rope"), (8192, 4096, 128, 128, "resid"), (4100, 8192, 192, 64, "rope"), (16384, 2048, 64, 128, "relu"),
    (8000, 4224, 128, 64, "resid"),                                       # the product's kernel normalises its own tiles
    (4096, 8192, 128, 128, "both"),                                       # rotation and residual update: two launches again
    (300, 512, 256, 128, "rope"), (32, 2048, 1024, 128, "resid"), (5, 256, 128, 64, "relu"),   # two launches
])
def test_matmul_with_the_producer_as_its_epilogue(ctx, m, n, k, d, variant):
    """tsattn_matmul_i8 with an epilogue is the product followed by tsattn_rope_normalize_rows on it: the same bytes, the
    same scales, the same updated residual, whichever way the library does it."""
    rng = np.random.default_rng(m * 7 + n + k)
    H = n // d
    a, w = dev(rand_i8(rng, (m, k)).view(np.uint8)), dev(rand_i8(rng, (n, k)).view(np.uint8))
    kw = {}
    if variant in ("rope", "both"):
        rope = dev(orc.fill_rope(d, 64))
        pos = dev(rng.integers(-1, 70, m).astype(np.int32))              # out-of-table positions are clamped
        kw = dict(pos=pos, rope=rope, scale_mult=0.37, rope_heads=max(1, H // 2), scale_heads=(H // 4, max(1, H // 4)))
    elif variant == "relu":
        kw = dict(relu=True, row_major_scale=True)
    resid0 = rng.standard_normal((m, n)).astype(np.float32)
    if variant in ("resid", "both"):
        r1, r2 = dev(resid0), dev(resid0)
        kw = dict(kw, resid=r1, resid_scale=0.011)
    got_q, got_s = ctx.matmul_normalize(a, w, H, capi.I8, **kw)
    sums = ctx.matmul_i8(a, w, mode=capi.MM_I32_PLANES)
    if variant in ("resid", "both"):
        kw = dict(kw, resid=r2, resid_scale=0.011)
    want_q, want_s = ctx.rope_normalize_rows(sums, H, capi.I8, **kw)
    torch.cuda.synchronize()
    assert torch.equal(got_q, want_q)
    assert torch.equal(got_s, want_s)
    if variant in ("resid", "both"):
        assert torch.equal(r1, r2)
