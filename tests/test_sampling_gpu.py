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


def test_prevent_eos_and_sampled_generation():
    name = "tiny_b"
    llm = H.llogos.Llogos(H.folder(name), dtype="float32", max_context=96, max_batch=3)
    prompts = [list(H.tokens(name, n, 60 + n)) for n in (40, 3, 9)]
    kw = dict(max_tokens=24, temperature=0.8, top_k=40, top_p=0.95, repetition_penalty=1.1, seed=1234, stop_tokens=())
    a = llm.generate(prompts, **kw).tokens
    assert a == llm.generate(prompts, **kw).tokens                      # a fixed seed repeats
    assert a != llm.generate(prompts, **dict(kw, seed=99)).tokens
    # every sampled token is one the plain sampler could draw: within the top 40 of the plain logits
    cfg, w = H.plain(name)
    for p, toks in zip(prompts, a):
        logits = pm.forward(cfg, w, p + toks)
        for i, t in enumerate(toks):
            row = logits[len(p) + i - 1].copy()
            assert t in np.argsort(-row)[:60]
    banned = a[0][0]
    b = llm.generate([prompts[0]], max_tokens=8, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0,
                     stop_tokens=(banned,), prevent_eos=True).tokens[0]
    assert len(b) == 8 and banned not in b


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
