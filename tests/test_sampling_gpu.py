"""The device sampler against the plain sampler with the same uniform numbers, and the
reference's own sampler vectors (tests/Daisi.Llogos.Tests/Inference/SamplerTests.cs)."""
import importlib

import numpy as np
import pytest
import torch

import gpu_helpers as H
import plain_model as pm

pytestmark = pytest.mark.gpu
S = importlib.import_module("daisi-llogos_amd.sampling")
DEV = "cuda:0"


def _draw(logits, params, us, histories=None):
    """One row per uniform number: the same logits sampled with each u."""
    logits = np.asarray(logits, dtype=np.float32)
    rows = torch.tensor(np.tile(logits, (len(us), 1)), device=DEV)
    sampler = S.Sampler(params)
    sampler.uniforms = lambda requests, indices: list(us)
    if histories is None:
        histories = [[]] * len(us)
    return sampler.sample(rows, list(range(len(us))), [0] * len(us), histories).cpu().tolist()


def _plain(logits, params, us, history=()):
    return [pm.sample(logits, float(np.float32(u)), temperature=params.temperature, top_k=params.top_k,
                      top_p=params.top_p, repetition_penalty=params.repetition_penalty,
                      frequency_penalty=params.frequency_penalty, presence_penalty=params.presence_penalty,
                      min_p=params.min_p, typical_p=params.typical_p, penalty_count=params.penalty_count,
                      min_keep=params.min_keep, penalize_newline=params.penalize_newline, history=history)
            for u in us]


def test_reference_vectors():
    us = np.random.default_rng(0).random(1000).astype(np.float32)
    off = dict(top_k=0, top_p=1.0, repetition_penalty=1.0)
    assert _draw([1., 5., 3., 2.], S.GenerationParams(temperature=0), [0.5]) == [1]
    lo = _draw([2., 1., .5, .1], S.GenerationParams(temperature=0.1, **off), us)
    hi = _draw([2., 1., .5, .1], S.GenerationParams(temperature=2.0, **off), us)
    assert lo.count(0) > 900 and hi.count(0) < 600
    tk = _draw([5., 4., 3., 2., 1., 0., -1., -2.], S.GenerationParams(temperature=1.0, top_k=3, top_p=1.0,
                                                                       repetition_penalty=1.0), us)
    assert set(tk) == {0, 1, 2}
    tp = _draw([10., 1., 0., -1.], S.GenerationParams(temperature=1.0, top_k=0, top_p=0.5, repetition_penalty=1.0), us[:500])
    assert tp.count(0) > 400
    pen = _draw([3., 3., 3., 3.], S.GenerationParams(temperature=0, repetition_penalty=2.0), [0.5], [[0, 1]])
    assert pen[0] >= 2
    eq = _draw([1.] * 5, S.GenerationParams(temperature=1.0, **off), [0.05, 0.25, 0.45, 0.65, 0.85])
    assert eq == [0, 1, 2, 3, 4]                                        # equal logits: index order


@pytest.mark.parametrize("opts", [
    dict(temperature=0.8, top_k=0, top_p=1.0, repetition_penalty=1.0),
    dict(temperature=0.8, top_k=40, top_p=0.95, repetition_penalty=1.1),            # the reference's defaults
    dict(temperature=1.3, top_k=7, top_p=0.6, repetition_penalty=1.0, min_keep=3),
    dict(temperature=0.7, top_k=0, top_p=0.9, repetition_penalty=1.3, frequency_penalty=0.2, presence_penalty=0.4,
         penalty_count=5),
    dict(temperature=1.0, top_k=50, top_p=1.0, repetition_penalty=1.0, min_p=0.1),
    dict(temperature=1.0, top_k=0, top_p=1.0, repetition_penalty=1.0, typical_p=0.6),
    dict(temperature=0.9, top_k=30, top_p=0.8, repetition_penalty=1.0, typical_p=0.7, min_p=0.02),
    dict(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.5, penalize_newline=True),
])
def test_pipeline_equals_the_plain_sampler(opts):
    rng = np.random.default_rng(1)
    params = S.GenerationParams(**opts)
    V = 1531                                                            # no power of two
    history = [3, 10, 10, 77, 3, 3, 1500, 13, 200, 41]
    for trial in range(3):
        logits = (rng.standard_normal(V) * 2.5).astype(np.float32)
        logits[history] += 3.0                                          # so that penalties decide something
        us = rng.random(64).astype(np.float32)
        got = _draw(logits, params, us, [history] * len(us))
        want = _plain(logits, params, us, history)
        same = sum(g == w for g, w in zip(got, want))
        # a draw within float rounding of a boundary of the cumulative sum may fall either way
        assert same >= len(us) - 1, (opts, got, want)


def test_large_vocabulary_and_batch_rows_are_independent():
    rng = np.random.default_rng(2)
    V, R = 128256, 6
    logits = torch.tensor((rng.standard_normal((R, V)) * 3).astype(np.float32), device=DEV)
    params = S.GenerationParams(temperature=0.9, top_k=40, top_p=0.95, repetition_penalty=1.0, seed=5)
    sampler = S.Sampler(params)
    all_rows = sampler.sample(logits, list(range(R)), [3] * R).cpu().tolist()
    alone = [sampler.sample(logits[i:i + 1], [i], [3]).item() for i in range(R)]
    assert all_rows == alone
    assert all_rows == sampler.sample(logits, list(range(R)), [3] * R).cpu().tolist()    # same seed, same draws
    other = S.Sampler(S.GenerationParams(temperature=0.9, top_k=40, top_p=0.95, repetition_penalty=1.0, seed=6))
    draws = [other.sample(logits, list(range(R)), [i] * R).cpu().tolist() for i in range(8)]
    assert len({tuple(d) for d in draws}) > 1
    for row, tok in zip(logits.cpu().numpy(), all_rows):
        assert tok in np.argsort(-row)[:40]


TINY_B_RUN = dict(max_tokens=24, temperature=0.8, seed=1234, stop_tokens=())      # 3 prompts of 40 / 3 / 9 tokens


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("filters", [dict(top_k=0, top_p=1.0, repetition_penalty=1.0),            # temperature alone
                                     dict(top_k=40, top_p=0.95, repetition_penalty=1.1)],          # the reference's defaults
                         ids=["temperature", "defaults"])
def test_sampled_generation_draw_by_draw(dtype, filters):
    """Three prompts of 40, 3 and 9 tokens, 24 tokens each at temperature 0.8 with a fixed seed, through the
    entry point; then every generated token again from the plain sampler on the plain logits of the
    same context with the same uniform number (seed, request, index of the token).  float32: the same
    token, but for at most one a sequence whose uniform number lies within rounding of a boundary of
    the cumulative sum.  bfloat16: the logits differ by roundings, which moves every boundary of the
    cumulative sum a little, and on the flat distributions of random weights (384 tokens of nearly
    equal weight) a third of the draws then falls to a neighbour; so every token must be one the
    plain sampler chooses among, and the uniform number must lie within `slack` of the part of
    [0, 1) that draws it there: twice the bound on the logits over the temperature, which is how far
    a difference of that size in every logit can move a cumulative sum; where the candidates are
    drawn in descending order (top-k, top-p), two parts more, since candidates of nearly equal weight
    change places in that order."""
    rng_mod = importlib.import_module("daisi-llogos_amd.sampling.rng")
    name = "tiny_b"
    llm = H.llogos.Llogos(H.folder(name), dtype=dtype, max_context=96, max_batch=3)
    prompts = [list(H.tokens(name, n, 60 + n)) for n in (40, 3, 9)]
    kw = dict(TINY_B_RUN, **filters)
    got = llm.generate(prompts, **kw).tokens
    assert [len(t) for t in got] == [24, 24, 24]
    assert got == llm.generate(prompts, **kw).tokens                    # a fixed seed repeats
    assert got != llm.generate(prompts, **dict(kw, seed=99)).tokens
    cfg, w = H.plain(name)
    slack = 0.0 if dtype == "float32" else 2 * H.tol(dtype, name) / kw["temperature"]
    same_all, worst = 0, 0.0
    for r, (p, toks) in enumerate(zip(prompts, got)):
        logits = pm.forward(cfg, w, p + toks)
        same = 0
        for i, t in enumerate(toks):
            cands, parts = [], {}
            u = rng_mod.uniform(kw["seed"], r, i)
            want = pm.sample(logits[len(p) + i - 1], u, temperature=kw["temperature"],
                             top_k=kw["top_k"], top_p=kw["top_p"], repetition_penalty=kw["repetition_penalty"],
                             history=(p + toks[:i]), candidates_out=cands, intervals_out=parts)
            assert t in cands, (dtype, r, i, t, want)
            same += t == want
            lo, hi = parts[t]
            worst = max(worst, lo - u, u - hi)
            if dtype == "bfloat16":
                room = slack + (2 * max(b - a for a, b in parts.values()) if kw["top_k"] or kw["top_p"] < 1 else 0.0)
                assert lo - room <= u < hi + room, (r, i, t, want, u, lo, hi, room)
        if dtype == "float32":
            assert same >= len(toks) - 1, (r, same)
        same_all += same
    print(f"{dtype} {filters}: {same_all} of 72 tokens are the plain sampler's; the uniform number lies at most "
          f"{worst:.4f} outside the drawn token's part (allowed {slack:.4f})")


def test_prevent_eos():
    """A stop token that would be drawn first: without prevent_eos nothing is generated; with it the token can
    not be drawn and the request runs to its last token.  (With temperature 0 and no penalty the reference
    takes its greedy short cut before it looks at PreventEOS, Daisi.Llogos/Inference/Sampler.cs:31-53, and so
    does this sampler: the option then changes nothing.)"""
    name = "tiny_b"
    llm = H.llogos.Llogos(H.folder(name), dtype="float32", max_context=96, max_batch=3)
    prompt = list(H.tokens(name, 40, 100))
    kw = dict(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.05)
    first = llm.generate([prompt], max_tokens=1, stop_tokens=(), **kw).tokens[0][0]
    assert llm.generate([prompt], max_tokens=8, stop_tokens=(first,), **kw).tokens[0] == []
    b = llm.generate([prompt], max_tokens=8, stop_tokens=(first,), prevent_eos=True, **kw).tokens[0]
    assert len(b) == 8 and first not in b
    greedy = dict(kw, repetition_penalty=1.0)
    first = llm.generate([prompt], max_tokens=1, stop_tokens=(), **greedy).tokens[0][0]
    assert llm.generate([prompt], max_tokens=8, stop_tokens=(first,), prevent_eos=True, **greedy).tokens[0] == []


def test_more_than_eight_banned_ids():
    """Twelve stop tokens that may not be drawn: the twelve largest logits of every row are
    theirs, the thirteenth must win (greedy) and no banned id is ever sampled."""
    rng = np.random.default_rng(8)
    V, R = 500, 5
    logits = rng.standard_normal((R, V)).astype(np.float32)
    banned = [int(t) for t in rng.choice(V, 12, replace=False)]
    logits[:, banned] += 20.0
    dev = torch.tensor(logits, device="cuda:0")
    K = importlib.import_module("daisi-llogos_amd.ops.kernels")
    work = K.sample_prepare(dev, None, None, 1.0, 0.0, 0.0, 1.0, False, banned).cpu().numpy()
    assert np.isneginf(work[:, banned]).all()
    keep = np.ones(V, bool); keep[banned] = False
    assert np.array_equal(work[:, keep], logits[:, keep])
    assert np.array_equal(K.argmax(torch.tensor(work, device="cuda:0")).cpu().numpy(),
                          np.where(keep, logits, -np.inf).argmax(1))
    with pytest.raises(K.KernelError, match="at most 64"):
        K.sample_prepare(dev, None, None, 1.0, 0.0, 0.0, 1.0, False, list(range(65)))
    params = S.GenerationParams(temperature=0.9, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=3, prevent_eos=True)
    sampler = S.Sampler(params, stop_tokens=banned)
    for i in range(20):
        drawn = sampler.sample(dev, list(range(R)), [i] * R).cpu().numpy()
        assert not set(drawn.tolist()) & set(banned)


def test_sampled_generation_draws_what_the_plain_sampler_draws():
    """Three prompts of 40 / 3 / 9 tokens, 24 new tokens each at temperature 0.8 with a fixed
    seed, in float32: along the engine's own token history, every token is the one the plain
    sampler draws from the plain logits with the same uniform number (the stream depends on
    seed, request and token index alone)."""
    rng_mod = importlib.import_module("daisi-llogos_amd.sampling.rng")
    name = "tiny_b"
    llm = H.llogos.Llogos(H.folder(name), dtype="float32", max_context=96, max_batch=3)
    prompts = [list(H.tokens(name, n, 60 + n)) for n in (40, 3, 9)]
    opts = dict(temperature=0.8, top_k=40, top_p=0.95, repetition_penalty=1.1)
    got = llm.generate(prompts, max_tokens=24, seed=1234, stop_tokens=(), **opts).tokens
    cfg, w = H.plain(name)
    differ = 0
    for r, (p, toks) in enumerate(zip(prompts, got)):
        logits = pm.forward(cfg, w, p + toks)
        for i, t in enumerate(toks):
            u = rng_mod.uniform(1234, r, i)
            want = pm.sample(logits[len(p) + i - 1], u, history=p + toks[:i], **opts)
            differ += int(want != t)
    assert differ == 0


def _every_way(rows, us, **opts):
    """Tokens drawn with the head of the order alone where that decides, with every row sorted
    whole by many blocks, and with every row sorted by its own block."""
    K = importlib.import_module("daisi-llogos_amd.ops.kernels")
    p = S.GenerationParams(**opts)
    out = []
    for order in ("head", "whole", "single"):
        work = K.sample_prepare(rows, None, None, 1.0, 0.0, 0.0, p.temperature, True)
        u = torch.tensor(np.asarray(us, dtype=np.float32), device=DEV)
        out.append(K.sample_pipeline(work, u, p.top_k, p.top_p, p.min_p, p.typical_p, p.min_keep, order=order).cpu().tolist())
    return out


def _peaked_rows(rng, R, V, spread):
    """Rows like a language model's: a few likely tokens, a long tail `spread` units wide."""
    rows = rng.standard_normal((R, V)).astype(np.float32) * spread
    for r in range(R):
        rows[r, rng.integers(0, V, 30)] += rng.random(30).astype(np.float32) * 4 * spread
    return rows


def _intervals(row, u_count, temperature, top_k, top_p, min_p=0.0, min_keep=1, **_):
    """The pipeline without typical-p in float64, vectorised for a large vocabulary: for every
    token the interval of uniform numbers that draws it (empty for tokens that are cut)."""
    work = row.astype(np.float64) / temperature
    order = np.lexsort((np.arange(len(work)), -work))
    n = top_k if 0 < top_k < len(work) else len(work)
    keep = max(min_keep, 1)
    if 0 < min_p < 1 and n > keep:
        n = max(keep, int((work[order[:n]] >= work[order[0]] + np.log(min_p)).sum()))
    cand = order[:n]
    p = np.exp(work[cand] - work[cand[0]])
    p /= p.sum()
    if 0 < top_p < 1:
        cut = np.nonzero((np.cumsum(p) > top_p) & (np.arange(n) + 1 >= keep))[0]
        if len(cut):
            cand, p = cand[:cut[0] + 1], p[:cut[0] + 1] / p[:cut[0] + 1].sum()
    hi = np.cumsum(p)
    lo_all, hi_all = np.ones(len(work)), np.zeros(len(work))
    lo_all[cand], hi_all[cand] = hi - p, hi
    return lo_all, hi_all


HEAD_OPTS = [
    dict(temperature=0.7, top_k=40, top_p=0.9),
    dict(temperature=0.7, top_k=0, top_p=0.9),
    dict(temperature=1.0, top_k=0, top_p=1.0),
    dict(temperature=1.0, top_k=0, top_p=0.98, min_p=0.001),
    dict(temperature=0.9, top_k=2048, top_p=1.0, min_keep=100),
    dict(temperature=0.9, top_k=3000, top_p=0.95),                      # more than the head holds: sorted whole
    dict(temperature=0.8, top_k=500, top_p=0.9, typical_p=0.8),
    dict(temperature=0.8, top_k=0, top_p=0.9, typical_p=0.8),           # typical-p over the vocabulary: sorted whole
]


@pytest.mark.parametrize("opts", HEAD_OPTS)
@pytest.mark.parametrize("V,spread", [(128256, 2.0), (151936, 0.5), (5000, 3.0)])
def test_the_head_of_the_order_decides_as_the_whole_order_does(opts, V, spread):
    """Rows like a language model's, with equal values, banned halves and the ends of the range
    of uniform numbers.  Both ways must draw the same tokens; a small vocabulary is compared with
    the plain sampler, a large one with the intervals of the cumulative distribution in float64:
    the uniform number lies in the drawn token's interval, within what float32 sums of 10^5 terms
    can be off (1e-5)."""
    rng = np.random.default_rng(V + int(opts["top_k"]))
    R = 12
    rows = _peaked_rows(rng, R, V, spread)
    rows[1, 7] = rows[1, 9] = rows[1].max() + 1.0                       # equal values at the top
    rows[2, rng.integers(0, V, V // 2)] = -np.inf                       # half of the row banned
    rows[3] = np.round(rows[3] * 2) / 2                                 # many equal values everywhere
    us = rng.random(R).astype(np.float32)
    us[4], us[5] = 0.0, np.float32(1.0 - 2 ** -24)                      # the ends of the range
    head, whole, single = _every_way(torch.tensor(rows, device=DEV), us, repetition_penalty=1.0, **opts)
    assert whole == single                                              # the same order, the same sums
    # a draw within float rounding of a boundary of the cumulative sum may fall either way
    assert sum(a != b for a, b in zip(head, whole)) <= 1, (head, whole)
    if V <= 5000:
        p = S.GenerationParams(repetition_penalty=1.0, **opts)
        want = [_plain(rows[r], p, [us[r]])[0] for r in range(R)]
        assert sum(a != b for a, b in zip(head, want)) <= 1, (head, want)
    elif "typical_p" not in opts:
        off = 0
        for r in range(R):
            lo, hi = _intervals(rows[r], us[r], **opts)
            off += not (lo[head[r]] - 1e-5 <= us[r] <= hi[head[r]] + 1e-5)
        assert off <= 1, (opts, head)


def test_rows_the_head_cannot_hold():
    """Every logit equal (one bin holds the row), a flat row of which top-p needs nine tenths, a
    row whose largest is infinite: the whole order decides, and gives what the plain sampler gives."""
    V = 20000
    us = [0.0, 0.3, 0.77, 0.999]
    for row, opts in ((np.ones(V, np.float32), dict(temperature=1.0, top_k=0, top_p=0.9)),
                      (np.ones(V, np.float32), dict(temperature=1.0, top_k=50, top_p=1.0)),
                      (np.linspace(0, 0.01, V).astype(np.float32), dict(temperature=1.0, top_k=0, top_p=0.9)),
                      (np.linspace(0, 100, V).astype(np.float32), dict(temperature=1.0, top_k=0, top_p=1.0))):
        rows = torch.tensor(np.tile(row, (len(us), 1)), device=DEV)
        head, whole, single = _every_way(rows, us, repetition_penalty=1.0, **opts)
        p = S.GenerationParams(repetition_penalty=1.0, **opts)
        assert head == whole == single == _plain(row, p, us), opts
    inf_row = np.zeros(V, np.float32)
    inf_row[5] = np.inf
    rows = torch.tensor(np.tile(inf_row, (2, 1)), device=DEV)
    head, whole, single = _every_way(rows, [0.2, 0.8], temperature=1.0, top_k=40, top_p=0.9, repetition_penalty=1.0)
    assert head == whole == single


def test_candidates_far_below_the_largest():
    """A low temperature spreads the candidates over a hundred units (coarse bins), and a row
    may have fewer tokens of probability above 0 than top-k or min_keep ask for: the head then
    holds every token that can be drawn."""
    rng = np.random.default_rng(11)
    V = 50000
    us = [0.0, 0.41, 0.93, 0.9999]
    wide = (rng.standard_normal(V) * 3).astype(np.float32)
    few = np.full(V, -np.inf, np.float32)
    few[[3, 77, 4000, 9, 12]] = [1.0, 0.5, 0.2, -200.0, -90.0]
    steep = (-np.arange(V) * 0.5).astype(np.float32)                    # one token per coarse bin, then exact zeros
    for row, opts in ((wide, dict(temperature=0.1, top_k=40, top_p=0.95)),
                      (wide, dict(temperature=0.05, top_k=0, top_p=1.0)),
                      (wide, dict(temperature=0.1, top_k=1000, top_p=1.0, min_p=1e-30)),
                      (few, dict(temperature=1.0, top_k=40, top_p=0.9)),
                      (few, dict(temperature=1.0, top_k=0, top_p=1.0, min_keep=20)),
                      (steep, dict(temperature=1.0, top_k=0, top_p=0.999)),
                      (steep, dict(temperature=1.0, top_k=500, top_p=1.0, typical_p=0.9))):
        rows = torch.tensor(np.tile(row, (len(us), 1)), device=DEV)
        head, whole, single = _every_way(rows, us, repetition_penalty=1.0, **opts)
        p = S.GenerationParams(repetition_penalty=1.0, **opts)
        assert head == whole == single == _plain(row, p, us), opts


def test_zeros_of_either_sign_are_equal_logits():
    """-0.0 and +0.0 compare equal, so among them the lower id comes first, as among other equal
    logits (rounded or penalised logits can hold both)."""
    row = np.array([0.0, -0.0, 0.0, -0.0, -0.0, 0.0, -3.0, 1.0] * 40, np.float32)
    us = [0.02, 0.2, 0.4, 0.6, 0.8, 0.97]
    rows = torch.tensor(np.tile(row, (len(us), 1)), device=DEV)
    for opts in (dict(temperature=1.5, top_k=0, top_p=1.0), dict(temperature=1.0, top_k=100, top_p=0.9),
                 dict(temperature=0.7, top_k=0, top_p=0.8, min_p=0.2)):
        head, whole, single = _every_way(rows, us, repetition_penalty=1.0, **opts)
        p = S.GenerationParams(repetition_penalty=1.0, **opts)
        assert head == whole == single == _plain(row, p, us), opts
