"""bin/trace_run as a user runs it: a subprocess fed with JSON steps, logits files out."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import gpu_helpers as H

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(model, dtype, steps, out_dir, max_tokens):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    return p.stdout.split("\n")


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_replay_of_two_batches(tmp_path, dtype):
    name = "tiny_b"
    vocab = 384
    a, b, c = H.tokens(name, 70, 1), H.tokens(name, 9, 2), H.tokens(name, 40, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": list(range(66))},
                                {"id": "b", "tokens": b[:8], "want": [7]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": [a[66]], "want": [0]},
                                {"id": "b", "tokens": [b[8]], "want": []}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": [a[67]], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": [a[68]], "want": [0]}], "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": c, "want": [0, 39]}], "end": ["c"]},
    ]
    out = str(tmp_path / "out")
    lines = _run(H.folder(name), dtype, steps, out, max_tokens=192)     # a: 128, b: 64; then c: 64
    assert [l for l in lines if l] == [f"done {i}" for i in range(5)]
    assert sorted(os.listdir(out)) == ["0.f32", "1.f32", "3.f32", "4.f32"]   # nothing wanted in step 2

    def read(step):
        return np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, vocab)
    pa, pb, pc = H.plain_logits(name, a), H.plain_logits(name, b), H.plain_logits(name, c)
    H.close(read(0), np.concatenate([pa[:66], pb[7:8]]), dtype, "step 0", config=name)
    H.close(read(1), pa[66:67], dtype, "step 1", config=name)
    H.close(read(3), pa[68:69], dtype, "step 3", config=name)
    H.close(read(4), pc[[0, 39]], dtype, "step 4", config=name)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["tiny_c", "tiny_d"])
def test_the_same_requests_whole_token_by_token_and_in_unequal_batches(tmp_path, name, dtype):
    """Three requests replayed three ways through the program: each alone and whole; each alone
    with its last 32 tokens one by one; and as batches of unequal lengths whose shorter requests
    end earlier, a second batch taking the slots of the first.  Every way against the plain
    implementation, and the ways against each other."""
    import tiny_configs as tc
    vocab = tc.ALL[name]["vocab_size"]
    reqs = {"a": H.tokens(name, 100, 11), "b": H.tokens(name, 45, 12), "c": H.tokens(name, 70, 13)}
    plain = {k: H.plain_logits(name, v) for k, v in reqs.items()}

    def replay(steps, max_tokens, tag):
        out = str(tmp_path / tag)
        lines = _run(H.folder(name), dtype, steps, out, max_tokens)
        assert [l for l in lines if l] == [f"done {s['step']}" for s in steps]
        got = {k: np.full((len(v), vocab), np.nan) for k, v in reqs.items()}
        fed = {k: 0 for k in reqs}
        for s in steps:
            rows = np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(-1, vocab) if any(e["want"] for e in s["entries"]) else None
            o = 0
            for e in s["entries"]:
                for w_ in e["want"]:
                    got[e["id"]][fed[e["id"]] + w_] = rows[o]
                    o += 1
                fed[e["id"]] += len(e["tokens"])
        return got

    # 1. whole, one request after the other
    steps = [{"step": i, "entries": [{"id": k, "tokens": list(v), "want": list(range(len(v)))}], "end": [k]}
             for i, (k, v) in enumerate(reqs.items())]
    whole = replay(steps, 128, "whole")
    # 2. the last 32 tokens one by one
    steps, n = [], 0
    for k, v in reqs.items():
        cut = len(v) - 32
        steps.append({"step": n, "entries": [{"id": k, "tokens": list(v[:cut]), "want": list(range(cut))}], "end": []}); n += 1
        for t in range(cut, len(v)):
            steps.append({"step": n, "entries": [{"id": k, "tokens": [v[t]], "want": [0]}], "end": [k] if t == len(v) - 1 else []}); n += 1
    single = replay(steps, 128, "single")
    # 3. unequal batches: a and b start together with prompts of 60 and 40 tokens, then one token each; b ends
    #    first; then c and a copy of b ("b2") as a second batch in the slots and pages that came back
    steps, n = [], 0
    steps.append({"step": n, "entries": [{"id": "a", "tokens": list(reqs["a"][:60]), "want": list(range(60))},
                                         {"id": "b", "tokens": list(reqs["b"][:40]), "want": list(range(40))}], "end": []}); n += 1
    for t in range(40):
        entries = [{"id": "a", "tokens": [reqs["a"][60 + t]], "want": [0]}]
        if t < 5:
            entries.append({"id": "b", "tokens": [reqs["b"][40 + t]], "want": [0]})
        steps.append({"step": n, "entries": entries, "end": (["b"] if t == 4 else []) + (["a"] if t == 39 else [])}); n += 1
    steps.append({"step": n, "entries": [{"id": "c", "tokens": list(reqs["c"][:69]), "want": list(range(69))}], "end": []}); n += 1
    steps.append({"step": n, "entries": [{"id": "c", "tokens": [reqs["c"][69]], "want": [0]}], "end": ["c"]}); n += 1
    batched = replay(steps, 192, "batched")
    tol = 2e-5 if dtype == "float32" else H.tol(dtype, name)
    for k in reqs:
        for way, got in (("whole", whole), ("token by token", single), ("batched", batched)):
            assert not np.isnan(got[k]).any(), (k, way)
            H.close(got[k], plain[k], dtype, f"{name} {k} {way}", config=name)
        assert np.abs(whole[k] - single[k]).max() <= tol and np.abs(whole[k] - batched[k]).max() <= tol


def test_replay_refuses_more_than_the_cache_holds(tmp_path):
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": list(range(65)), "want": []}], "end": []}]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", H.folder("tiny_a"),
           "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    p = subprocess.run(cmd, input=json.dumps(steps[0]) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode != 0 and "pages" in p.stderr


def test_command_line_generates_and_benchmarks():
    """The command line as a subprocess: greedy generation prints token ids, --bench the
    reference's block (Daisi.Llogos.Cli/Program.cs:292-296)."""
    import plain_model as pm
    name = "tiny_b"
    cfg, w = H.plain(name)
    prompt = list(H.tokens(name, 12, 77))
    cmd = [sys.executable, "-m", "daisi-llogos_amd", "--model", H.folder(name), "--prompt", " ".join(map(str, prompt)),
           "-n", "6", "-t", "0", "--repeat-penalty", "1.0", "--dtype", "float32", "--max-context", "64"]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    got = [int(t) for t in p.stdout.split()]
    want = pm.generate_greedy(cfg, w, prompt, 6, stop=set(cfg_eos(name)))
    assert got == want
    assert "prefill: 12 tokens" in p.stderr and "decode:" in p.stderr
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llogos"), "-m", H.folder(name), "--bench", "-n", "8",
                        "--prompt-len", "20", "--batch", "2", "--max-context", "64"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert "=== Benchmark Results ===" in p.stderr and "Prefill:" in p.stderr and "Decode:" in p.stderr
    assert "40 tokens" in p.stderr.split("Prefill:")[1].split("\n")[0].replace("    ", " ")


def cfg_eos(name):
    import tiny_configs as tc
    e = tc.ALL[name]["eos_token_id"]
    return e if isinstance(e, list) else [e]
