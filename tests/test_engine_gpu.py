"""The engine against the plain implementation, in float32 and in bfloat16: each request
alone and whole; the last 32 tokens one by one; batches of unequal lengths whose shorter
requests end earlier, one batch after another so that slots and pages are used again;
long decoding; the first tokens of a sequence; greedy generation through the entry point."""
import importlib

import numpy as np
import pytest
import torch

import gpu_helpers as H
import plain_model as pm
import tiny_configs as tc

K = importlib.import_module("daisi-llogos_amd.ops.kernels")

pytestmark = pytest.mark.gpu
CONFIGS = ["tiny_a", "tiny_b", "tiny_c", "tiny_w", "tiny_d"]


def _np(t):
    return t.detach().cpu().double().numpy()


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", CONFIGS)
def test_whole_requests(name, dtype):
    eng = H.engine(name, dtype)
    for n, seed in ((5, 1), (17, 2), (1, 3), (32, 4), (100, 5)):
        toks = H.tokens(name, n, seed)
        s = eng.alloc_slot()
        got = _np(eng.step([(s, toks)], want="all"))
        eng.free_slot(s)
        H.close(got, H.plain_logits(name, toks), dtype, f"{name} whole n={n}", config=name)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", CONFIGS)
def test_last_32_tokens_one_by_one(name, dtype):
    eng = H.engine(name, dtype)
    toks = H.tokens(name, 120, 7)
    want = H.plain_logits(name, toks)
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, toks[:88])], want="all"))]
    for t in toks[88:]:
        rows.append(_np(eng.step([(s, [t])], want="last")))
    got = np.concatenate(rows)
    H.close(got, want, dtype, f"{name} decode", config=name)
    # the same positions in one step: cutting changes nothing beyond rounding
    s2 = eng.alloc_slot()
    whole = _np(eng.step([(s2, toks)], want="all"))
    tol = 1e-5 if dtype == "float32" else H.tol(dtype, name)
    assert np.abs(whole - got).max() <= tol


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", CONFIGS)
def test_unequal_batches_one_after_another(name, dtype):
    """Batches of unequal prompts; shorter requests end earlier; the pool is so small that
    the next batch must take the slots and pages the last one gave back."""
    eng = H.engine(name, dtype, max_tokens=64 * 5, n_slots=4)
    plans = [
        [(5, 16), (17, 3), (1, 9), (32, 12)],       # (prompt length, decoded tokens) per request
        [(40, 24), (3, 5), (9, 30)],
        [(64, 2), (63, 1), (60, 30)],          # 2 + 1 + 2 pages: the pool is full at the end
    ]
    seed = 20
    for plan in plans:
        reqs = []
        for n_prompt, n_dec in plan:
            seed += 1
            toks = H.tokens(name, n_prompt + n_dec, seed)
            reqs.append(dict(toks=toks, n_prompt=n_prompt, slot=eng.alloc_slot(), rows=[], fed=0))
        assert sorted(r["slot"] for r in reqs) == list(range(len(reqs)))       # slots are used again
        out = eng.step([(r["slot"], r["toks"][:r["n_prompt"]]) for r in reqs], want="all")
        o = 0
        for r in reqs:
            r["rows"].append(_np(out[o:o + r["n_prompt"]]))
            o += r["n_prompt"]
            r["fed"] = r["n_prompt"]
        live = list(reqs)
        while live:
            for r in [r for r in live if r["fed"] == len(r["toks"])]:
                eng.free_slot(r["slot"])                                         # ends earlier than the others
                live.remove(r)
            if not live:
                break
            out = eng.step([(r["slot"], [r["toks"][r["fed"]]]) for r in live], want="last")
            for i, r in enumerate(live):
                r["rows"].append(_np(out[i:i + 1]))
                r["fed"] += 1
        for r in reqs:
            H.close(np.concatenate(r["rows"]), H.plain_logits(name, r["toks"]), dtype,
                    f"{name} batch request of {len(r['toks'])}", config=name)
        assert eng.cache.live_slots == [] and eng.cache.free_pages() == [5] * len(eng.cache.groups)


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_batch_composition_and_slot_do_not_change_float_results(dtype):
    """A request alone in slot 0 and the same request last in a batch, in another slot and in
    other pages: equal logits (each row's arithmetic is its own)."""
    name = "tiny_a"
    eng = H.engine(name, dtype, n_slots=8)
    toks = H.tokens(name, 70, 31)
    s = eng.alloc_slot()
    alone = [_np(eng.step([(s, toks[:50])], want="all"))] + [_np(eng.step([(s, [t])])) for t in toks[50:]]
    eng.free_slot(s)
    others = [H.tokens(name, n, 40 + n) for n in (90, 3, 66)]
    slots = [eng.alloc_slot() for _ in range(4)]
    out = eng.step([(slots[i], o) for i, o in enumerate(others)] + [(slots[3], toks[:50])],
                   want=[[], [], [], list(range(50))])
    mixed = [_np(out)]
    for i, t in enumerate(toks[50:]):
        batch = [(slots[j], [others[j][(i + j) % len(others[j])]]) for j in range(3)] + [(slots[3], [t])]
        mixed.append(_np(eng.step(batch, want=[[], [], [], [0]])))
    a, b = np.concatenate(alone), np.concatenate(mixed)
    if dtype == "float32":
        assert np.array_equal(a, b), f"max difference {np.abs(a - b).max()}"
    else:
        # the bfloat16 engine picks its matrix-product kernel by the number of rows (library
        # product above 64 rows), so sums are ordered differently: equal within rounding, and
        # the single-token steps, which use one kernel at every batch size, exactly
        assert np.abs(a - b).max() <= H.tol(dtype, name)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["tiny_c", "tiny_w", "tiny_d"])
def test_long_decoding(name, dtype):
    """300 positions, most of them decoded one by one: crosses page borders, and in the
    windowed configuration pages leave the window and are given back meanwhile."""
    eng = H.engine(name, dtype, max_tokens=64 * 6, n_slots=1)
    toks = H.tokens(name, 300, 9)
    want = H.plain_logits(name, toks)
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, toks[:3])], want="all"))]
    for t in toks[3:]:
        rows.append(_np(eng.step([(s, [t])], want="last")))
    H.close(np.concatenate(rows), want, dtype, f"{name} long decode", config=name)
    if name == "tiny_w":
        assert eng.cache.free_pages()[1] > eng.cache.free_pages()[0]           # the window group gave pages back


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["tiny_d", "tiny_w"])
def test_a_context_of_thousands_of_positions(name, dtype):
    """2,300 positions: a prompt of 36 pages in one step, a second one continued across a page's
    end beside it, then single tokens for both (page tables wider than one bucket of the
    captured steps, many blocks along the context and their merge)."""
    eng = H.engine(name, dtype, max_tokens=64 * 80, n_slots=2)
    a, b = H.tokens(name, 2300, 21), H.tokens(name, 2200, 22)
    pa, pb = H.plain_logits(name, a), H.plain_logits(name, b)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    got = _np(eng.step([(sa, a[:2290]), (sb, b[:2000])], want=[[0, 63, 64, 2289], [1999]]))
    H.close(got, np.stack([pa[0], pa[63], pa[64], pa[2289], pb[1999]]), dtype, f"{name}: long prompts", config=name)
    got = _np(eng.step([(sa, [a[2290]]), (sb, b[2000:2190])], want=[[0], [0, 47, 189]]))
    H.close(got, np.stack([pa[2290], pb[2000], pb[2047], pb[2189]]), dtype, f"{name}: a token beside a continued prompt", config=name)
    for t in range(2291, 2296):
        got = _np(eng.step([(sa, [a[t]]), (sb, [b[t - 101]])], want="last"))
        H.close(got, np.stack([pa[t], pb[t - 101]]), dtype, f"{name}: token {t}", config=name)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", CONFIGS)
def test_first_tokens(name, dtype):
    eng = H.engine(name, dtype)
    toks = H.tokens(name, 6, 13)
    want = H.plain_logits(name, toks)
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, [t])], want=[[0]])) for t in toks]               # from the very first token on
    H.close(np.concatenate(rows), want, dtype, f"{name} first tokens", config=name)
    s2 = eng.alloc_slot()
    assert eng.step([(s2, toks[:2])], want=None) is None                       # nothing wanted: no logits
    got = _np(eng.step([(s2, toks[2:])], want=[[3, 0]]))                       # places in the asked order
    H.close(got, want[[5, 2]], dtype, f"{name} wanted places", config=name)


@pytest.mark.parametrize("name", ["tiny_a", "tiny_d"])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_window_and_sinks_as_run_time_strategy(name, dtype):
    cfg, w = H.plain(name)
    toks = H.tokens(name, 100, 17)
    want = pm.forward(cfg, w, list(toks), window=24, sinks=3)
    eng = H.engine(name, dtype, attention_window=24, attention_sinks=3)
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, toks[:70])], want="all"))] + [_np(eng.step([(s, [t])])) for t in toks[70:]]
    H.close(np.concatenate(rows), want, dtype, "window 24 sinks 3", config=name)
    assert np.abs(want - H.plain_logits(name, toks)).max() > 1e-3              # the window matters here


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["layer_8b", "layer_14b"])
def test_layer_sizes_of_large_models(name, dtype):
    """Two layers of the Llama-3.1-8B layer sizes (hidden 4096, 32/8 heads of 128, feed-forward
    14336) and one of the Qwen3-14B sizes (hidden 5120, 40/8 heads with their norm, feed-forward
    17408): whole, the last tokens one by one, and an unequal batch, against the plain
    implementation."""
    eng = H.engine(name, dtype, max_tokens=64 * 12, n_slots=3)
    a, b, c = H.tokens(name, 150, 1), H.tokens(name, 70, 2), H.tokens(name, 3, 3)
    pa, pb, pc = (H.plain_logits(name, t) for t in (a, b, c))
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, a[:140])], want="all"))] + [_np(eng.step([(s, [t])])) for t in a[140:]]
    H.close(np.concatenate(rows), pa, dtype, f"{name}: prompt then tokens", config=name)
    eng.free_slot(s)
    slots = [eng.alloc_slot() for _ in range(3)]
    out = _np(eng.step([(slots[0], a[:100]), (slots[1], b[:66]), (slots[2], c[:2])], want="all"))
    H.close(out, np.concatenate([pa[:100], pb[:66], pc[:2]]), dtype, f"{name}: unequal batch", config=name)
    out = _np(eng.step([(slots[0], [a[100]]), (slots[1], [b[66]]), (slots[2], [c[2]])], want="last"))
    H.close(out, np.stack([pa[100], pb[66], pc[2]]), dtype, f"{name}: one token each", config=name)
    eng.free_slot(slots[2])
    out = _np(eng.step([(slots[0], a[101:150]), (slots[1], [b[67]])], want=[[48], [0]]))
    H.close(out, np.stack([pa[149], pb[67]]), dtype, f"{name}: a continued prompt beside a single token", config=name)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["tiny_c", "layer_8b"])
def test_batches_of_more_than_64_sequences(name, dtype):
    """100 sequences with prompts of 3 to 9 tokens in one step, then one token each while a third
    of them ends early: beyond the batch sizes whose steps are captured, where the products take
    other kernels (the library's, and the few-row product in its form for 65 to 128 rows)."""
    n = 100
    base = [H.tokens(name, 13, 40 + j) for j in range(5)]
    plain = [H.plain_logits(name, b) for b in base]
    eng = H.engine(name, dtype, max_tokens=64 * n, n_slots=n)
    slots = [eng.alloc_slot() for _ in range(n)]
    seq, plen = [i % 5 for i in range(n)], [3 + i % 7 for i in range(n)]
    out = _np(eng.step([(slots[i], base[seq[i]][:plen[i]]) for i in range(n)], want="last"))
    H.close(out, np.stack([plain[seq[i]][plen[i] - 1] for i in range(n)]), dtype, f"{name}: 100 prompts", config=name)
    live = list(range(n))
    for t in range(4):
        out = _np(eng.step([(slots[i], [base[seq[i]][plen[i] + t]]) for i in live], want="last"))
        H.close(out, np.stack([plain[seq[i]][plen[i] + t] for i in live]), dtype, f"{name}: token {t} of {len(live)} sequences", config=name)
        if t == 0:
            for i in live[::3]:
                eng.free_slot(slots[i])
            live = [i for i in live if i % 3]
    assert len(live) == 66


def test_step_errors():
    eng = H.engine("tiny_a", "float32", max_tokens=128, n_slots=2)
    s = eng.alloc_slot()
    with pytest.raises(H.llogos.StepError, match="token id"):
        eng.step([(s, [256])])
    with pytest.raises(H.llogos.StepError, match="at least one token"):
        eng.step([(s, [])])
    with pytest.raises(H.llogos.StepError, match="twice"):
        eng.step([(s, [1]), (s, [2])])
    with pytest.raises(H.llogos.StepError, match="outside"):
        eng.step([(s, [1, 2])], want=[[2]])
    with pytest.raises(H.llogos.CacheError):
        eng.step([(5, [1])])
    with pytest.raises(H.llogos.CacheFull):
        eng.step([(s, list(range(129)))])
    assert eng.cache.length(s) == 0 and eng.cache.free_pages() == [2]          # refused steps change nothing
    eng.step([(s, [1, 2, 3])])
    assert eng.cache.length(s) == 3


@pytest.mark.parametrize("name", ["tiny_b", "tiny_w", "layer_14b"])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_replayed_steps_equal_steps_launched_kernel_by_kernel(name, dtype):
    """Single-token steps replayed as a captured graph against the same steps launched kernel
    by kernel, bit for bit, replay after replay, with other work of the engine between the
    replays: prompts of other sequences, sequences that end, and a batch that shrinks and
    grows (another graph each)."""
    engines = [H.engine(name, dtype, max_tokens=64 * 24, n_slots=4, use_graphs=g) for g in (True, False)]
    assert engines[0].graphs is not None and engines[1].graphs is None
    rng = np.random.default_rng(3)
    vocab = tc.ALL[name]["vocab_size"]
    new = lambda n: [int(t) for t in rng.integers(0, vocab, n)]
    plan = [("prompt", 0, new(70)), ("prompt", 1, new(5))] + [("tokens", (0, 1), None)] * 6 + \
           [("prompt", 2, new(130))] + [("tokens", (0, 1, 2), None)] * 5 + [("end", 1, None)] + \
           [("tokens", (0, 2), None)] * 4 + [("prompt", 3, new(64))] + [("tokens", (3, 0, 2), None)] * 5
    slots = [{}, {}]
    for what, arg, toks in plan:
        outs = []
        step_tokens = new(len(arg)) if what == "tokens" else None
        for e, (eng, sl) in enumerate(zip(engines, slots)):
            if what == "prompt":
                sl[arg] = eng.alloc_slot()
                outs.append(eng.step([(sl[arg], toks)], want="last"))
            elif what == "end":
                eng.free_slot(sl.pop(arg))
            else:
                outs.append(eng.step([(sl[r], [t]) for r, t in zip(arg, step_tokens)], want="last"))
        if outs:
            assert torch.equal(outs[0], outs[1]), (what, arg)
    assert len(engines[0].graphs.graphs) >= 2


def test_replayed_steps_of_twenty_sequences():
    """The same with 20 sequences at the Qwen3-14B layer sizes, where the gate/up product takes
    the kernel whose operands go straight into LDS: its launches replay like the others'."""
    name, dtype, n = "layer_14b", "bfloat16", 20
    assert K.skinny_plan(n, 2 * tc.ALL[name]["intermediate_size"], tc.ALL[name]["hidden_size"])[0] == "strips"
    engines = [H.engine(name, dtype, max_tokens=64 * (n + 2), n_slots=n + 1, use_graphs=g) for g in (True, False)]
    rng = np.random.default_rng(4)
    vocab = tc.ALL[name]["vocab_size"]
    new = lambda k: [int(t) for t in rng.integers(0, vocab, k)]
    prompts = [new(3 + i % 4) for i in range(n)]
    slots = [[eng.alloc_slot() for _ in range(n)] for eng in engines]
    outs = [eng.step(list(zip(sl, prompts)), want="last") for eng, sl in zip(engines, slots)]
    assert torch.equal(outs[0], outs[1])
    extra = [None, None]
    for t in range(5):
        toks = new(n)
        outs = [eng.step([(s, [tok]) for s, tok in zip(sl, toks)], want="last") for eng, sl in zip(engines, slots)]
        assert torch.equal(outs[0], outs[1]), t
        if t == 1:                                       # other work between the replays
            p = new(40)
            for e, eng in enumerate(engines):
                extra[e] = eng.alloc_slot()
                eng.step([(extra[e], p)], want=None)
        if t == 2:
            for e, eng in enumerate(engines):
                eng.free_slot(extra[e])
    assert len(engines[0].graphs.graphs) >= 1


def test_captured_steps_are_dropped_and_made_again(monkeypatch):
    """More batch shapes than captured steps are kept: the least recently used one goes, and
    a shape that comes back is captured again; results stay those of uncaptured steps."""
    graph_mod = importlib.import_module("daisi-llogos_amd.engine.graph")
    monkeypatch.setattr(graph_mod, "MAX_GRAPHS", 2)
    name, dtype = "tiny_b", "bfloat16"
    engines = [H.engine(name, dtype, max_tokens=64 * 12, n_slots=6, use_graphs=g) for g in (True, False)]
    rng = np.random.default_rng(8)
    slots = [[eng.alloc_slot() for _ in range(5)] for eng in engines]
    for eng, sl in zip(engines, slots):
        eng.step([(s, list(H.tokens(name, 3 + i, 40 + i))) for i, s in enumerate(sl)], want=None)
    for batch in (1, 2, 3, 4, 5, 1, 3, 5, 2, 2, 4):
        toks = [int(t) for t in rng.integers(0, tc.ALL[name]["vocab_size"], batch)]
        outs = [eng.step([(s, [t]) for s, t in zip(sl[:batch], toks)], want="last") for eng, sl in zip(engines, slots)]
        assert torch.equal(outs[0], outs[1]), batch
        assert len(engines[0].graphs.graphs) <= 2


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_a_batch_that_shrinks_replays_a_few_captured_sizes(dtype):
    """19 sequences that end one after the other: the steps between two captured batch sizes
    run as the larger one with padding rows, which belong to no sequence; every sequence's
    logits are, bit for bit, those of uncaptured steps without padding, also for sequences that
    start in the slots and pages the ended ones gave back."""
    graph_mod = importlib.import_module("daisi-llogos_amd.engine.graph")
    name, n = "tiny_a", 19
    engines = [H.engine(name, dtype, max_tokens=64 * (n + 4), n_slots=n, use_graphs=g) for g in (True, False)]
    rng = np.random.default_rng(12)
    vocab = tc.ALL[name]["vocab_size"]
    new = lambda k: [int(t) for t in rng.integers(0, vocab, k)]
    prompts = [new(1 + (7 * i) % 11) for i in range(n)]
    slots = [[eng.alloc_slot() for _ in range(n)] for eng in engines]
    outs = [eng.step(list(zip(sl, prompts)), want="last") for eng, sl in zip(engines, slots)]
    assert torch.equal(outs[0], outs[1])
    live = list(range(n))
    while live:
        toks = new(len(live))
        outs = [eng.step([(sl[r], [t]) for r, t in zip(live, toks)], want="last") for eng, sl in zip(engines, slots)]
        assert torch.equal(outs[0], outs[1]), len(live)
        gone = live.pop(int(rng.integers(0, len(live))))
        for eng, sl in zip(engines, slots):
            eng.free_slot(sl[gone])
    sizes = {key[0] for key in engines[0].graphs.graphs}
    assert sizes <= set(graph_mod.BATCH_BUCKETS) and sizes == {graph_mod.bucket_batch(b) for b in range(1, n + 1)}
    # the slots and pages that came back, used again at a size with padding
    for eng in engines:
        assert eng.cache.live_slots == [] and len(set(eng.cache.free_pages())) == 1
    slots = [[eng.alloc_slot() for _ in range(10)] for eng in engines]
    prompts = [new(2 + i) for i in range(10)]
    for _ in range(3):
        outs = [eng.step(list(zip(sl, prompts)), want="last") for eng, sl in zip(engines, slots)]
        assert torch.equal(outs[0], outs[1])
        prompts = [[int(t)] for t in rng.integers(0, vocab, 10)]


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_a_step_can_take_its_tokens_from_the_device(dtype, graphs):
    """Single-token steps fed from an int32 vector on the device (in any order of rows) give
    bit for bit what the same tokens from the host give, replayed as a graph or not."""
    import torch
    name = "tiny_b"
    seqs = [list(H.tokens(name, n, 70 + n)) for n in (9, 70, 6)]
    outs = []
    for fed in (False, True):
        eng = H.engine(name, dtype, max_tokens=1024, n_slots=4, use_graphs=graphs)
        slots = [eng.alloc_slot() for _ in seqs]
        eng.step([(s, q[:-4]) for s, q in zip(slots, seqs)], want=None)
        got = []
        for k in range(4, 0, -1):
            toks = [q[-k] for q in seqs]
            if fed:
                # the tokens lie in another order in a longer vector, as after sequences have ended
                src = torch.tensor([7, toks[2], toks[0], 1, toks[1]], dtype=torch.int32, device="cuda:0")
                got.append(eng.step([(s, [0]) for s in slots], want="last", device_ids=(src, [2, 4, 1])))
            else:
                got.append(eng.step([(s, [t]) for s, t in zip(slots, toks)], want="last"))
        outs.append(_np(torch.stack(got)))
        if fed:
            with pytest.raises(H.llogos.StepError, match="rows"):
                eng.step([(s, [0]) for s in slots], device_ids=(src, [0, 1, 5]))
            with pytest.raises(H.llogos.StepError, match="one token"):
                eng.step([(slots[0], [0, 0])], device_ids=(src, [0]))
            with pytest.raises(H.llogos.StepError, match="int32"):
                eng.step([(slots[0], [0])], device_ids=(src.float(), [0]))
    assert np.array_equal(outs[0], outs[1])
    plain_rows = np.stack([np.stack([H.plain_logits(name, tuple(q))[len(q) - k] for q in seqs]) for k in range(4, 0, -1)])
    H.close(outs[1], plain_rows, dtype, "device-fed steps", config=name)


@pytest.mark.parametrize("temperature", [0.0, 0.7])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_generation_that_looks_ahead_gives_the_same_tokens(dtype, temperature):
    """The loop that starts a step before the host has read the last one's tokens against
    the loop that waits: same tokens, stop tokens honoured, every slot and page given back."""
    import torch
    name = "tiny_a"
    gen_mod = importlib.import_module("daisi-llogos_amd.engine.generate")
    prompts = [list(H.tokens(name, n, 90 + n)) for n in (5, 17, 1, 32, 8, 3)]
    eng = H.engine(name, dtype, max_tokens=64 * 8, n_slots=4)
    params = H.llogos.GenerationParams(max_tokens=20, temperature=temperature, top_k=0 if temperature == 0 else 20,
                                       top_p=1.0, repetition_penalty=1.0, seed=5, stop_tokens=())
    free = eng.cache.free_pages()
    base = gen_mod.Generator(eng, max_batch=4, synchronize=torch.cuda.synchronize, look_ahead=False).generate(prompts, params)
    # tokens that the requests draw at different times become stop tokens
    stops = tuple({base.tokens[0][3], base.tokens[1][9], base.tokens[4][0], base.tokens[5][19]})
    params = H.llogos.GenerationParams(max_tokens=20, temperature=temperature, top_k=0 if temperature == 0 else 20,
                                       top_p=1.0, repetition_penalty=1.0, seed=5, stop_tokens=stops)
    res = []
    for ahead in (False, True):
        g = gen_mod.Generator(eng, max_batch=4, synchronize=torch.cuda.synchronize, look_ahead=ahead)
        res.append(g.generate(prompts, params))
        assert eng.cache.live_slots == [] and eng.cache.free_pages() == free
    assert res[0].tokens == res[1].tokens and res[0].finish_reasons == res[1].finish_reasons
    assert "stop" in res[1].finish_reasons
    for toks, full, why in zip(res[1].tokens, base.tokens, res[1].finish_reasons):
        assert toks == full[:len(toks)] and (len(toks) == 20) == (why == "length")


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b"])
def test_greedy_generation_through_the_entry_point(name, dtype):
    cfg, w = H.plain(name)
    prompts = [list(H.tokens(name, n, 50 + n)) for n in (5, 17, 1, 32, 8)]
    llm = H.llogos.Llogos(H.folder(name), dtype=dtype, max_context=64, max_batch=3)
    res = llm.generate(prompts, max_tokens=16, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0,
                       stop_tokens=())
    assert res.batches == [[0, 1, 2], [3, 4]] and all(len(t) == 16 for t in res.tokens)
    for p, toks in zip(prompts, res.tokens):
        logits = pm.forward(cfg, w, p + toks)
        for i, t in enumerate(toks):
            row = logits[len(p) + i - 1]
            # the chosen token is the plain implementation's maximum, up to the dtype's rounding
            assert row.max() - row[t] <= (0 if dtype == "float32" else 2 * H.tol(dtype, name)), (name, dtype, i)
    # stop tokens end a sequence and are not emitted
    first = res.tokens[0]
    res2 = llm.generate([prompts[0]], max_tokens=16, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0,
                        stop_tokens=(first[4],))
    cut = first.index(first[4])
    assert res2.tokens[0] == first[:cut] and res2.finish_reasons == ["stop"]
    assert llm.engine.cache.live_slots == []
