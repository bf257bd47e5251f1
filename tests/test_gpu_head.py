"""GPU: the embedding sum, the final softmax with the greedy choice (ComputePrediction, gpt/train/cpu_infer.cpp:552-582) and
the sampled choice (SampleFromDistr, :585-599) through the C ABI against the oracle."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from tscale_amd import AttentionContext
    c = AttentionContext(0, max_seqs=1, max_heads=16, max_head_dim=128)
    yield c
    c.close()


dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_embed_rows_bit_exact(ctx):
    rng = np.random.default_rng(5)
    embed = rng.integers(-127, 128, (300, 256)).astype(np.int8)
    labels = rng.integers(-2, 302, (41, 3)).astype(np.int32)      # some empty slots on both sides
    want = orc.embed_rows(labels, embed, 0.0173)
    got = ctx.embed_rows(dev(labels), dev(embed.view(np.uint8)), 0.0173)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    one = ctx.embed_rows(dev(labels[:, 0].copy()), dev(embed.view(np.uint8)), 0.0173).cpu().numpy()
    assert np.array_equal(one, orc.embed_rows(labels[:, :1], embed, 0.0173))


@pytest.mark.parametrize("n_rows,n,planes", [(32, 50257, 1), (3, 1000, 4), (1, 7, 1)])
def test_softmax_rows_and_greedy_choice(ctx, n_rows, n, planes):
    rng = np.random.default_rng(n)
    parts = (rng.standard_normal((planes, n_rows, n)) * 3000).astype(np.int32)
    vec = parts.sum(axis=0).astype(np.int32)
    bias = rng.standard_normal(n).astype(np.float32)
    scale = 2e-3
    # the reference's own arithmetic (polynomial exp2, eight running sums); a single running float sum over 50k terms,
    # the oracle's other mode, is itself 1e-4 off
    want, want_arg = orc.softmax_rows(vec, scale, bias, exp2_mode=1)
    src = dev(parts if planes > 1 else vec)
    prob, arg = ctx.softmax_rows(src, scale, dev(bias))
    torch.cuda.synchronize()
    got = prob.cpu().numpy()
    assert np.array_equal(arg.cpu().numpy(), want_arg)
    big = want > 1e-30
    assert np.abs(got[big] / want[big] - 1).max() < 1e-4 and np.abs(got - want).max() < 5e-5
    assert np.abs(got.sum(axis=1) - 1).max() < 1e-4
    # the choice alone, without the probabilities and without a bias
    _, arg2 = ctx.softmax_rows(src, scale, None, want_prob=False)
    assert np.array_equal(arg2.cpu().numpy(), orc.softmax_rows(vec, scale, None)[1])


def test_softmax_rows_ties_and_negative_rows(ctx):
    tie = np.zeros((2, 600), dtype=np.int32)
    tie[0, [77, 300, 599]] = 9
    tie[1] = -40000
    prob, arg = ctx.softmax_rows(dev(tie), 1e-3)
    assert arg.cpu().numpy().tolist() == [77, 0]
    want, _ = orc.softmax_rows(tie, 1e-3)
    assert np.abs(prob.cpu().numpy() - want).max() < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("n_rows,n,temperature", [(8, 50257, 1.0), (32, 1000, 0.7), (3, 77, 2.5)])
def test_sample_rows_matches_the_oracle(ctx, n_rows, n, temperature):
    """SampleFromDistr on the device against the oracle, with the caller's random words and with the counter-based
    generator.  Scores are compared through the choice: a different index is accepted only where the oracle's own
    scores of the two indices are within rounding of each other (logf and log differ in the last bit between libm
    and the device)."""
    rng = np.random.default_rng(n)
    w = (rng.standard_normal((n_rows, n)) * 3).astype(np.float32)
    prob = np.exp(w - w.max(axis=1, keepdims=True)); prob = (prob / prob.sum(axis=1, keepdims=True)).astype(np.float32)
    prob[0, 5] = 0.0                                                     # never chosen
    words = rng.integers(0, 2**32, (n_rows, n), dtype=np.uint64).astype(np.uint32)
    dprob = torch.from_numpy(prob).cuda()
    for rnd, seed, offset in ((words, 0, 0), (None, 1313, 12345)):
        want = orc.sample_rows(prob, temperature, rnd=rnd, seed=seed, offset=offset)
        drnd = None if rnd is None else torch.from_numpy(rnd.view(np.int32)).cuda()
        got = ctx.sample_rows(dprob, temperature, rnd=drnd, seed=seed, offset=offset).cpu().numpy()
        for i in np.nonzero(got != want)[0]:
            r = rnd[i] if rnd is not None else np.array([orc.mix32(seed, offset + i * n + k) for k in range(n)], dtype=np.uint32)
            u = (r.astype(np.float64) + 0.5) / 2.0**32
            with np.errstate(divide="ignore"):
                score = np.log(prob[i].astype(np.float64)) / temperature - np.log(-np.log(u))
            assert abs(score[got[i]] - score[want[i]]) < 1e-5 * max(1.0, abs(score[want[i]])), (i, got[i], want[i])
        assert got[0] != 5


@pytest.mark.gpu
def test_sample_rows_argument_checks(ctx):
    from tscale_amd import capi
    prob = torch.full((2, 10), 0.1, dtype=torch.float32, device="cuda")
    with pytest.raises(capi.TsattnError):
        ctx.sample_rows(prob, 0.0)
    with pytest.raises(capi.TsattnError):
        ctx.sample_rows(prob, -1.0)
