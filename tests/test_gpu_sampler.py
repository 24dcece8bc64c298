"""Sampler on the GPU, through the C ABI, against the oracle with the same noise tensor."""
import pytest
import torch

import oracle
from nanovllm_amd import Sampler
from nanovllm_amd import sample as _sample
from nanovllm_amd import synthetic
from helpers import assert_sampled_like_oracle

pytestmark = pytest.mark.gpu

_mode = {"static": False}


def sample(*args, **kw):
    kw.setdefault("static_scratch", _mode["static"])
    return _sample(*args, **kw)


@pytest.fixture(autouse=True, params=[False, True], ids=["workspace", "static"])
def _scratch_mode(request):
    """Every test runs twice: through nva_sample (workspace tensor) and through nva_sample_static
    (records in the library's own array, what the engine's Sampler module calls)."""
    _mode["static"] = request.param
    yield
    _mode["static"] = False


def _check(case, dev):
    tok = sample(case.logits.to(dev), case.temperatures.to(dev), case.noise.to(dev))
    torch.cuda.synchronize()
    assert tok.dtype == torch.int64 and tok.shape == (case.logits.shape[0],)
    scores = oracle.sample_scores(case.logits, case.temperatures, case.noise)
    return assert_sampled_like_oracle(tok, scores)


@pytest.mark.parametrize("batch,temp", [(64, 0.6), (256, 0.6), (128, 1.0)])
def test_sampler_full_vocab(dev, batch, temp):
    """151,936-way vocabulary, the temperatures of the 0.6B bench and of the 8B stress."""
    case = synthetic.sampler_case(seed=batch, batch=batch, temperature=temp)
    differ = _check(case, dev)
    assert differ <= max(1, batch // 50)          # near-ties are rare


@pytest.mark.parametrize("batch,vocab", [(1, 1), (3, 7), (5, 2047), (4, 2048), (4, 2049), (2, 10001), (7, 33333)])
def test_sampler_ragged_vocab(dev, batch, vocab):
    case = synthetic.sampler_case(seed=vocab, batch=batch, vocab=vocab, temperature=0.9)
    _check(case, dev)


def test_sampler_mixed_temperatures_and_greedy_rows(dev):
    case = synthetic.sampler_case(seed=5, batch=32, vocab=50000)
    case.temperatures[:] = torch.linspace(0.2, 2.0, 32)
    case.temperatures[::4] = 0.0                               # greedy rows
    tok = sample(case.logits.to(dev), case.temperatures.to(dev), case.noise.to(dev)).cpu()
    want = oracle.sample(case.logits, case.temperatures, case.noise)
    greedy = case.temperatures == 0
    assert torch.equal(tok[greedy], case.logits.float().argmax(-1)[greedy])
    scores = oracle.sample_scores(case.logits, torch.where(greedy, torch.ones(32), case.temperatures), case.noise)
    assert_sampled_like_oracle(tok[~greedy], scores[~greedy])
    assert (tok == want).float().mean() > 0.9


def test_sampler_unit_noise_is_argmax_first_index_on_ties(dev):
    logits = torch.zeros(6, 5000, dtype=torch.bfloat16)
    logits[0, 4000] = logits[0, 123] = 3.0                     # exact tie: first index wins
    logits[1, 4999] = 1.0
    logits[2, 0] = 1.0
    logits[3, 2048] = logits[3, 2047] = 2.0
    ones = torch.ones(6, 5000)
    tok = sample(logits.to(dev), torch.full((6,), 0.7).to(dev), ones.to(dev)).cpu()
    assert tok.tolist() == [123, 4999, 0, 2047, 0, 0]
    assert torch.equal(tok, oracle.sample(logits, torch.full((6,), 0.7), ones))


def test_sampler_noise_clamp(dev):
    case = synthetic.sampler_case(seed=6, batch=8, vocab=3000)
    case.noise[:, 77] = 0.0                                    # clamped to 1e-10: wins
    tok = sample(case.logits.to(dev), case.temperatures.to(dev), case.noise.to(dev)).cpu()
    assert tok.tolist() == [77] * 8


def test_sampler_strided_logits(dev):
    case = synthetic.sampler_case(seed=7, batch=4, vocab=4001)
    wide = torch.zeros(4, 4104, dtype=torch.bfloat16)
    wide[:, :4001] = case.logits
    tok = sample(wide.to(dev)[:, :4001], case.temperatures.to(dev), case.noise.to(dev))
    scores = oracle.sample_scores(case.logits, case.temperatures, case.noise)
    assert_sampled_like_oracle(tok, scores)


def test_sampler_philox_mode_is_categorical_and_reproducible(dev):
    v, n, t = 12, 60000, 0.8
    row = torch.tensor([2.0, 1.0, 0.5, 0.0, -0.5, -1.0, 1.5, 0.25, -2.0, 0.75, -0.25, 1.25]).to(torch.bfloat16)
    logits = row.expand(n, v).contiguous().to(dev)
    temps = torch.full((n,), t, device=dev)
    a = sample(logits, temps, None, seed=11, offset=1).cpu()
    b = sample(logits, temps, None, seed=11, offset=1).cpu()
    c = sample(logits, temps, None, seed=11, offset=2).cpu()
    assert torch.equal(a, b) and not torch.equal(a, c)
    p = torch.softmax(row.double() / t, -1)
    for tok in (a, c):
        freq = torch.bincount(tok, minlength=v).double()
        chi2 = float(((freq - n * p) ** 2 / (n * p)).sum())
        assert chi2 < 40.0, chi2
    # the module interface draws fresh noise per call
    s = Sampler(seed=3)
    x, y = s(logits, temps).cpu(), s(logits, temps).cpu()
    assert x.shape == (n,) and not torch.equal(x, y)


@pytest.mark.parametrize("batch,vocab,scale", [(64, 151936, 2.0), (33, 4001, 1.0), (8, 50000, 4.0), (5, 7, 1.0),
                                               (16, 8192, 1.0), (16, 8193, 3.0), (3, 8192 * 66 + 5, 2.0)])
def test_sampler_in_kernel_draw_is_the_tree_of_inverse_cdf_draws(dev, batch, vocab, scale):
    """Without a noise tensor the token of row b is what the oracle's float64 tree of inverse-CDF
    draws yields from the same Philox uniforms.  The kernel sums in fp32, so rows whose uniform lies
    within rounding of an interval edge at some level may take the neighbouring branch; every other
    row must agree exactly, and no row may return a column of zero probability.  (The last case has
    more than 64 chunks per row: the row kernel then walks the chunk records in several rounds.)"""
    g = torch.Generator().manual_seed(vocab)
    logits = (torch.randn(batch, vocab, generator=g) * scale).to(torch.bfloat16)
    logits[0, : min(3, vocab - 1)] = float("-inf")           # leading columns that cannot be drawn
    temps = torch.linspace(0.5, 1.3, batch)
    seed, offset = 0x1234567811, 77
    tok = sample(logits.to(dev), temps.to(dev), None, seed=seed, offset=offset).cpu()
    want, margin = oracle.tree_draw(logits, temps, seed, offset)
    sure = margin > 2e-5
    assert int(sure.sum()) >= batch - max(1, batch // 16)
    assert torch.equal(tok[sure], want[sure]), (tok, want, margin)
    assert bool((logits[torch.arange(batch), tok].float() > float("-inf")).all())


def test_sampler_in_kernel_draw_edge_rows(dev):
    """Rows with a single finite logit (first, last, chunk edges) return it; a row of -inf returns 0."""
    vocab = 3 * 8192 + 17
    cols = [0, 7, 8, 2047, 2048, 8191, 8192, vocab - 1]
    logits = torch.full((len(cols) + 1, vocab), float("-inf"), dtype=torch.bfloat16)
    for r, c in enumerate(cols):
        logits[r, c] = -3.0
    temps = torch.full((len(cols) + 1,), 0.6)
    for offset in (1, 2, 3):
        tok = sample(logits.to(dev), temps.to(dev), None, seed=4, offset=offset).cpu()
        assert tok.tolist() == cols + [0]


def test_sampler_philox_mode_large_vocab_and_greedy(dev):
    """In-kernel noise on a wide, flat vocabulary: bucketed chi-square against the softmax, a
    dominant logit always wins, and temperature-0 rows are plain argmax."""
    v, n, t = 4096, 50000, 1.0
    g = torch.Generator().manual_seed(3)
    row = (torch.randn(v, generator=g) * 0.5).to(torch.bfloat16)
    logits = row.expand(n, v).contiguous().to(dev)
    tok = sample(logits, torch.full((n,), t, device=dev), None, seed=5, offset=9).cpu()
    p = torch.softmax(row.double() / t, -1)
    buckets = 64
    freq = torch.bincount(tok // (v // buckets), minlength=buckets).double()
    pb = p.view(buckets, -1).sum(-1)
    chi2 = float(((freq - n * pb) ** 2 / (n * pb)).sum())
    assert chi2 < 130.0, chi2                     # 63 dof: P(chi2 > 130) ~ 1e-6
    peaked = torch.zeros(8, 151936, dtype=torch.bfloat16)
    peaked[torch.arange(8), torch.arange(8) * 18000 + 7] = 60.0
    out = sample(peaked.to(dev), torch.full((8,), 0.6, device=dev), None, seed=1, offset=1).cpu()
    assert out.tolist() == [i * 18000 + 7 for i in range(8)]
    case = synthetic.sampler_case(seed=8, batch=16, vocab=151936)
    out = sample(case.logits.to(dev), torch.zeros(16, device=dev), None, seed=2, offset=3).cpu()
    assert torch.equal(out, case.logits.float().argmax(-1))
