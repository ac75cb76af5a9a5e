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
    H.close(read(0), np.concatenate([pa[:66], pb[7:8]]), dtype, "step 0")
    H.close(read(1), pa[66:67], dtype, "step 1")
    H.close(read(3), pa[68:69], dtype, "step 3")
    H.close(read(4), pc[[0, 39]], dtype, "step 4")


def test_replay_refuses_more_than_the_cache_holds(tmp_path):
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": list(range(65)), "want": []}], "end": []}]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", H.folder("tiny_a"),
           "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    p = subprocess.run(cmd, input=json.dumps(steps[0]) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode != 0 and "pages" in p.stderr
