"""The sampling kernels alone, against the plain sampler, at other sizes than the engine's."""
import numpy as np
import pytest
import torch

import plain

pytestmark = pytest.mark.gpu


def _logits(rows, vocab, seed, scale=3.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(rows, vocab, generator=g) * scale


@pytest.mark.parametrize("vocab", [1, 7, 256, 1000, 4097, 128256])
def test_argmax_lowest_index_among_equals(vocab):
    from llama_cu_amd.sampling import argmax
    l = _logits(5, vocab, vocab)
    if vocab > 6:
        l[1, 3] = l[1, vocab - 2] = 50.0            # equal maxima: the lower index wins
        l[2, vocab - 1] = 60.0
    got = argmax(l.cuda()).tolist()
    assert got == [plain.sample(r, 0.0, 1.0, 10 ** 9, 0.5) for r in l]


@pytest.mark.parametrize("vocab,temperature,top_p,top_k", [
    (50, 1.0, 1.0, 10 ** 9), (301, 0.8, 1.0, 10 ** 9), (1000, 0.7, 0.9, 10 ** 9), (1000, 1.3, 1.0, 5),
    (4097, 0.5, 0.5, 40), (128256, 0.8, 0.95, 50), (128256, 1.0, 1.0, 10 ** 9)])
def test_sample_kernel_matches_plain_sampler(vocab, temperature, top_p, top_k):
    """The same uniform number gives the same token, except where it falls within rounding
    of the boundary between two tokens (then either is accepted)."""
    from llama_cu_amd.sampling import sample_rows
    rows = 24
    l = _logits(rows, vocab, 17 + vocab)
    l[3, 5 % vocab] = l[3, 11 % vocab]              # equal logits inside a row
    rng = np.random.default_rng(vocab)
    u = [0.0, 0.999999] + [float(x) for x in rng.random(rows - 2)]
    got = sample_rows(l.cuda(), [temperature] * rows, [top_p] * rows, [top_k] * rows, u).tolist()
    for r in range(rows):
        want = plain.sample(l[r], temperature, top_p, top_k, u[r])
        if got[r] != want:
            _assert_draw_within_rounding(l[r], temperature, top_p, top_k, u[r], got[r])


@pytest.mark.parametrize("rows", [3, 40])
def test_equal_logits_across_the_parts_of_a_long_row(rows):
    """A long row is cut into parts, one workgroup each.  With few distinct values thousands of
    logits are equal, spread over all parts: the draw is the m-th of them in index order, as a
    stable sort has them; with and without a cut at top_k that falls among equals."""
    from llama_cu_amd.sampling import sample_rows
    vocab = 70001
    g = torch.Generator().manual_seed(rows)
    l = (torch.randn(rows, vocab, generator=g) * 2.0).round() * 0.5        # steps of a half: a few dozen values
    rng = np.random.default_rng(rows)
    u = [0.0, 0.999999] + [float(x) for x in rng.random(rows - 2)]
    for top_p, top_k in ((1.0, 10 ** 9), (0.9, 5000), (1.0, 37)):
        got = sample_rows(l.cuda(), [0.7] * rows, [top_p] * rows, [top_k] * rows, u).tolist()
        for r in range(rows):
            want = plain.sample(l[r], 0.7, top_p, top_k, u[r])
            if got[r] != want:
                _assert_draw_within_rounding(l[r], 0.7, top_p, top_k, u[r], got[r])


def _assert_draw_within_rounding(logits, temperature, top_p, top_k, u, token, tol=2e-6):
    """``token`` is the right answer for a number within ``tol`` of ``u``: in the sorted
    order of llama.cu/src/op/random_sample/sample.cuh:186-207 its span of the cumulative
    weights, widened by ``tol`` of the limit, holds ``u * limit``."""
    x = logits.double()
    order = torch.sort(x, descending=True, stable=True).indices
    w = torch.exp((x[order] - x[order][0]) / temperature)
    c = torch.cumsum(w, 0)
    k = min(top_k, x.numel())
    limit = min(top_p * float(c[-1]), float(c[k - 1]))
    i = int((order == token).nonzero()[0])
    lo = float(c[i - 1]) if i else 0.0
    assert lo - tol * limit <= u * limit <= float(c[i]) + tol * limit, (token, i, u, lo / limit, float(c[i]) / limit)


def test_sample_frequencies_follow_the_cut_softmax():
    from llama_cu_amd.sampling import sample_rows
    vocab, n = 40, 20000
    l = _logits(1, vocab, 5, scale=1.5)[0]
    rng = np.random.default_rng(1)
    u = [float(x) for x in rng.random(n)]
    T, k = 0.9, 7
    got = sample_rows(l.repeat(n, 1).cuda(), [T] * n, [1.0] * n, [k] * n, u).cpu().numpy()
    p = torch.softmax(l.double() / T, 0).numpy()
    keep = np.argsort(-p)[:k]
    q = np.zeros(vocab); q[keep] = p[keep]; q /= q.sum()
    freq = np.bincount(got, minlength=vocab) / n
    assert np.abs(freq - q).max() < 0.015
    assert freq[[i for i in range(vocab) if i not in keep]].sum() == 0


def test_sample_frequencies_with_a_top_p_cut_inside_the_support():
    """top_p cuts the cumulative weights of the sorted tokens at ``top_p`` of their total
    (llama.cu/src/op/random_sample/sample.cuh:71-87: the drawn number is scaled by
    ``min(top_p * c[n-1], c[top_k-1])``): tokens wholly below the cut keep their weight, the token
    that the cut falls into keeps only the part below the cut, and nothing beyond it is ever drawn.
    (The usual nucleus rule would keep that token whole: the frequencies tell the two apart.)"""
    from llama_cu_amd.sampling import sample_rows
    vocab, n, T, top_p = 30, 40000, 1.1, 0.62
    l = _logits(1, vocab, 11, scale=1.2)[0]
    rng = np.random.default_rng(3)
    u = [float(x) for x in rng.random(n)]
    got = sample_rows(l.repeat(n, 1).cuda(), [T] * n, [top_p] * n, [10 ** 9] * n, u).cpu().numpy()
    p = torch.softmax(l.double() / T, 0).numpy()
    order = np.argsort(-p, kind="stable")
    c = np.cumsum(p[order])
    q = np.zeros(vocab)
    below = 0.0
    for rank, tok in enumerate(order):
        q[tok] = max(0.0, min(c[rank], top_p) - below) / top_p
        below = c[rank]
    cut = int(np.searchsorted(c, top_p))                       # the rank the cut falls into
    assert 2 <= cut < vocab - 3                                 # strictly inside the support
    part = q[order[cut]] * top_p / p[order[cut]]
    assert 0.15 < part < 0.85                                   # a real part of that token, neither none nor all of it
    freq = np.bincount(got, minlength=vocab) / n
    assert np.abs(freq - q).max() < 0.01
    assert freq[order[cut + 1:]].sum() == 0                     # nothing beyond the cut
    whole = p[order[cut]] / c[cut]                              # what the token would get if it were kept whole
    assert abs(freq[order[cut]] - q[order[cut]]) < 0.01 < abs(whole - q[order[cut]])


def test_per_row_parameters_and_sampler_mix():
    from llama_cu_amd.sampling import Sampler, SamplingParams, uniform
    l = _logits(4, 500, 9)
    params = [SamplingParams(), SamplingParams(temperature=0.8, seed=3), SamplingParams(temperature=1.0, top_k=1),
              SamplingParams(temperature=1.2, top_p=0.7, top_k=20, seed=5)]
    keys = [(0, 10), (1, 11), (2, 12), (3, 13)]
    got = Sampler().sample(l.cuda(), params, keys)
    for r in range(4):
        p = params[r]
        want = plain.sample(l[r], p.temperature, p.top_p, min(p.top_k, 10 ** 9), uniform(p.seed, *keys[r]))
        assert got[r] == want


def test_the_chosen_tokens_log_probability():
    """``token_logprobs`` against ``torch.log_softmax`` in 64-bit, on rows of a vocabulary that is no power of two with a
    stride of its own, one row sharp (a logit far above the rest) and one flat; and through the engine: the tokens of an
    engine made with ``logprobs`` come with the plain model's log-probabilities."""
    from llama_cu_amd.sampling import token_logprobs
    g = torch.Generator().manual_seed(3)
    rows, vocab = 7, 128256 + 3
    buf = torch.randn(rows, vocab + 5, generator=g) * 3.0
    buf[2, 777] = 60.0
    buf[4, :] = 0.25
    logits = buf.cuda()[:, :vocab]
    tokens = torch.tensor([0, vocab - 1, 777, 5, 9, 100000, 31], dtype=torch.int32)
    got = token_logprobs(logits, tokens.cuda()).cpu().double()
    want = torch.log_softmax(buf[:, :vocab].double(), dim=-1)[torch.arange(rows), tokens.long()]
    assert float((got - want).abs().max()) < 1e-4, (got, want)
    assert abs(float(got[2])) < 1e-6 and abs(float(got[4]) + float(torch.log(torch.tensor(float(vocab))))) < 1e-4
    assert torch.isnan(token_logprobs(logits[:1], torch.tensor([vocab], dtype=torch.int32).cuda())).all()


@pytest.mark.parametrize("run_ahead", [False, True])
def test_an_engine_made_with_logprobs_hands_them_out_with_its_tokens(run_ahead):
    import common
    import plain
    from llama_cu_amd.engine.engine import Engine
    from llama_cu_amd.sampling import SamplingParams
    folder = common.make_folder(common.TINY_A, seed=5, dtype=torch.float32)
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_seqs=4, run_ahead=run_ahead, logprobs=True)
    prompts = list(common.random_requests(256, [9, 30], seed=2).values())
    params = [SamplingParams(), SamplingParams(temperature=0.9, seed=4)]
    ids = [engine.add_request(p, sp, 6, ignore_eos=True) for p, sp in zip(prompts, params)]
    got = {i: [] for i in ids}
    while not engine.idle:
        for o in engine.step():
            if o.token is not None:
                assert o.logprob is not None
                got[o.req].append((o.token, o.logprob))
    cfg, w = plain.load_folder(folder)
    for rid, prompt in zip(ids, prompts):
        toks = list(prompt)
        assert len(got[rid]) == 6
        for tok, lp in got[rid]:
            want = torch.log_softmax(plain.forward(cfg, w, toks)[-1], dim=-1)[tok]
            assert abs(lp - float(want)) < 1e-3, (rid, len(toks), lp, float(want))
            toks.append(tok)
