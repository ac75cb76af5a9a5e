"""The generation loop's decisions, with a stand-in engine: batching, stop tokens, sequences
that end earlier, slots given back and used again."""
import importlib

import numpy as np
import pytest

gen = importlib.import_module("daisi-llogos_amd.engine.generate")
kvc = importlib.import_module("daisi-llogos_amd.cache.kv_cache")
base = importlib.import_module("daisi-llogos_amd.parts.base")
params_mod = importlib.import_module("daisi-llogos_amd.sampling.params")
GenerationParams = params_mod.GenerationParams

VOCAB = 50


class FakeEngine:
    """Next token = (sum of the sequence's tokens so far) % VOCAB; the cache is the real
    bookkeeping without device memory."""

    def __init__(self, max_tokens=64 * 8, n_slots=2):
        self.cache = kvc.Cache([(base.KVSpec(1, 16), None)], [None], max_tokens, rt=None, n_slots=n_slots)
        self.sums = {}
        self.log = []

    def alloc_slot(self):
        s = self.cache.alloc_slot()
        self.sums[s] = 0
        return s

    def free_slot(self, s):
        self.cache.free_slot(s)
        del self.sums[s]

    def step(self, entries, want="last"):
        assert want == "last"
        slots = [s for s, _ in entries]
        lens = [self.cache.length(s) + len(t) for s, t in entries]
        self.cache.reserve(slots, lens)
        self.cache.commit(slots, lens)
        self.log.append([(s, len(t)) for s, t in entries])
        out = np.full((len(entries), VOCAB), -1.0, dtype=np.float32)
        for i, (s, t) in enumerate(entries):
            self.sums[s] += sum(t)
            out[i, self.sums[s] % VOCAB] = 1.0
        return out


class AheadEngine(FakeEngine):
    """The same, able to take a step's tokens from the ids a sampler left behind."""
    takes_device_ids = True

    def step(self, entries, want="last", device_ids=None):
        if device_ids is not None:
            ids, rows = device_ids
            assert all(len(t) == 1 for _, t in entries) and len(rows) == len(entries)
            self.fed = getattr(self, "fed", 0) + len(entries)
            entries = [(s, [int(ids[i])]) for (s, _), i in zip(entries, rows)]
        return super().step(entries, want)


class ArgmaxSampler:
    def sample(self, logits, requests, indices, histories):
        self.last = (list(requests), list(indices))
        return np.argmax(logits, axis=-1)


def expected(prompt, n, stops=()):
    seq, out = list(prompt), []
    for _ in range(n):
        t = sum(seq) % VOCAB
        if t in stops:
            return out, "stop"
        out.append(t)
        seq.append(t)
    return out, "length"


def test_plan_batches():
    assert gen.plan_batches([5, 5, 5, 5, 5], 10, 2, 100) == [[0, 1], [2, 3], [4]]
    # pages: 70 + 10 -> 2 pages each, the pool has 5
    assert gen.plan_batches([70, 70, 70], 10, 8, 5) == [[0, 1], [2]]
    with pytest.raises(ValueError, match="cache"):
        gen.plan_batches([70, 600], 10, 8, 5)
    with pytest.raises(ValueError, match="empty"):
        gen.plan_batches([3, 0], 10, 8, 5)


def test_unequal_prompts_lengths_and_stops():
    eng = FakeEngine()
    g = gen.Generator(eng, max_batch=8)
    prompts = [[1, 2, 3], [7], [4, 4, 4, 4, 4, 4], [9, 9]]
    stops = (13, 30)
    res = g.generate(prompts, GenerationParams.greedy(max_tokens=12, stop_tokens=stops), sampler=ArgmaxSampler())
    for p, toks, why in zip(prompts, res.tokens, res.finish_reasons):
        want, reason = expected(p, 12, stops)
        assert toks == want and why == reason
        assert not set(toks) & set(stops)                              # a stop token is never emitted
    assert {"stop", "length"} <= set(res.finish_reasons) or len(set(res.finish_reasons)) == 1
    assert res.prompt_tokens == 12 and res.generated_tokens == sum(len(t) for t in res.tokens)
    assert eng.cache.live_slots == [] and eng.cache.free_pages() == [8]
    # the first step holds all prompts whole, later steps one token for each live sequence
    assert eng.log[0] == [(0, 3), (1, 1), (2, 6), (3, 2)]
    assert all(n == 1 for step in eng.log[1:] for _, n in step)
    sizes = [len(step) for step in eng.log]
    assert sizes == sorted(sizes, reverse=True)                        # the batch only shrinks


def test_ended_sequences_leave_and_slots_are_used_again():
    eng = FakeEngine(n_slots=2)
    g = gen.Generator(eng, max_batch=2)
    prompts = [[1], [2, 2], [3, 3, 3], [5], [8, 1]]
    res = g.generate(prompts, GenerationParams.greedy(max_tokens=5, stop_tokens=(4,)), sampler=ArgmaxSampler())
    assert res.batches == [[0, 1], [2, 3], [4]]
    for p, toks, why in zip(prompts, res.tokens, res.finish_reasons):
        assert (toks, why) == expected(p, 5, (4,))
    assert {s for step in eng.log for s, _ in step} == {0, 1}           # two slots serve five requests
    assert eng.cache.slots.n_slots == 2 and eng.cache.live_slots == []


def test_max_tokens_zero_and_one():
    eng = FakeEngine()
    g = gen.Generator(eng)
    res = g.generate([[1, 2]], GenerationParams.greedy(max_tokens=0), sampler=ArgmaxSampler())
    assert res.tokens == [[]] and eng.log == []
    res = g.generate([[1, 2]], GenerationParams.greedy(max_tokens=1, stop_tokens=()), sampler=ArgmaxSampler())
    assert res.tokens == [[3]] and len(eng.log) == 1                    # no step after the last token


def test_sampler_sees_request_and_token_index():
    eng = FakeEngine()
    s = ArgmaxSampler()
    gen.Generator(eng).generate([[1], [2], [3]], GenerationParams.greedy(max_tokens=3, stop_tokens=(4,)), sampler=s)
    # request 1 (prompt [2]) draws 2, then 4 = stop: at the last step only requests 0 and 2 are live
    assert s.last == ([0, 2], [2, 2])


def test_slots_are_given_back_when_a_step_fails():
    eng = FakeEngine(max_tokens=64 * 2)
    g = gen.Generator(eng)

    class Boom(Exception):
        pass

    def bad(entries, want="last"):
        raise Boom()
    eng.step = bad
    with pytest.raises(Boom):
        g.generate([[1, 2, 3]], GenerationParams.greedy(max_tokens=4), sampler=ArgmaxSampler())
    assert eng.cache.live_slots == []


def test_params_follow_the_reference_defaults():
    p = GenerationParams()
    assert (p.max_tokens, p.temperature, p.top_k, p.top_p, p.repetition_penalty) == (256, 0.8, 40, 0.95, 1.1)
    assert (p.penalty_count, p.min_keep, p.typical_p, p.min_p) == (64, 1, 1.0, 0.0)
    assert not p.is_greedy and GenerationParams.greedy().is_greedy
    assert not GenerationParams(temperature=0).is_greedy               # penalties still apply
    with pytest.raises(ValueError):
        GenerationParams(temperature=-1)


def test_uniform_stream_is_per_request():
    rng = importlib.import_module("daisi-llogos_amd.sampling.rng")
    a = [rng.uniform(7, 2, i) for i in range(50)]
    assert a == [rng.uniform(7, 2, i) for i in range(50)]
    assert all(0 <= u < 1 for u in a) and len(set(a)) == 50
    assert a != [rng.uniform(8, 2, i) for i in range(50)] and a != [rng.uniform(7, 3, i) for i in range(50)]
    us = [rng.uniform(1, r, i) for r in range(40) for i in range(50)]
    assert abs(sum(us) / len(us) - 0.5) < 0.02


@pytest.mark.parametrize("max_tokens", [1, 2, 3, 12])
def test_looking_ahead_changes_no_result(max_tokens):
    """With the host one step behind, a request that drew a stop token has run one step too
    many; tokens, finish reasons and the slots given back are the same as without."""
    prompts = [[1, 2, 3], [7], [4, 4, 4, 4, 4, 4], [9, 9], [3], [5, 6]]
    stops = (13, 30, 14)
    p = GenerationParams.greedy(max_tokens=max_tokens, stop_tokens=stops)
    results = []
    for engine in (FakeEngine(n_slots=4), AheadEngine(n_slots=4)):
        g = gen.Generator(engine, max_batch=4)
        seen = []
        res = g.generate(prompts, p, sampler=ArgmaxSampler(), on_token=lambda r, t: seen.append((r, t)))
        for i, pr in enumerate(prompts):
            want, why = expected(pr, max_tokens, stops)
            assert res.tokens[i] == want and res.finish_reasons[i] == why
        assert sorted(seen) == sorted((i, t) for i, toks in enumerate(res.tokens) for t in toks)
        assert not engine.cache.live_slots and not engine.sums          # every slot came back
        assert engine.cache.free_pages() == [engine.cache.n_pages]
        results.append(res)
    assert results[0].generated_tokens == results[1].generated_tokens
    # the engine that looks ahead also stepped every stop token it drew, unless that token would
    # have been the request's last anyway; it never stepped a request past its last token
    ahead = AheadEngine(n_slots=4)
    res = gen.Generator(ahead, max_batch=4).generate(prompts, p, sampler=ArgmaxSampler())
    single = getattr(ahead, "fed", 0)
    want_single = 0
    for toks, why in zip(res.tokens, res.finish_reasons):
        n = len(toks)
        want_single += n - 1 if why == "length" else n + (1 if n + 1 < max_tokens else 0)
    assert single == want_single


def test_recent_tokens_are_the_tail_of_prompt_and_generated():
    for prompt, generated, count in (([1, 2, 3], [4, 5], 2), ([1, 2, 3], [4, 5], 4), ([1, 2, 3], [4, 5], 10),
                                     ([1, 2, 3], [], 0), ([], [7], 3), ([1, 2, 3], [4, 5], 5), ([1, 2, 3], [4, 5], -1)):
        whole = prompt + generated
        assert gen.recent_tokens(prompt, generated, count) == (whole[-count:] if count > 0 else whole)


def test_prevent_eos_refuses_more_stop_tokens_than_the_kernel_bans():
    """Stop tokens beyond what one sampling call can ban are an error, not silently drawable."""
    sampler_mod = importlib.import_module("daisi-llogos_amd.sampling.sampler")
    params = GenerationParams(temperature=0.7, prevent_eos=True)
    sampler_mod.Sampler(params, stop_tokens=range(64))
    with pytest.raises(ValueError, match="at most 64"):
        sampler_mod.Sampler(params, stop_tokens=range(65))
    sampler_mod.Sampler(GenerationParams(temperature=0.7), stop_tokens=range(100))      # only stops, nothing to ban
