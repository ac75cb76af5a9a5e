"""Trace replay: feed given token ids through the engine step by step and write logits.
It samples nothing and has no model code of its own: it drives Engine.step.

Analogues in the reference are tests that dump or compare logits per step
(tests/Daisi.Llogos.Tests/Chat/LogitDumpTest.cs:55-94, LayerByLayerCompareTest.cs:61-110);
this is a program.

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, <out>/<step>.f32 holds the logits at the wanted
places, in the order of the entries and of `want`, little-endian float32 [wanted, vocab].
After every step `done <step>` is printed and flushed."""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, Iterable, TextIO

import numpy as np

from .step import Engine


class TraceError(ValueError):
    pass


def replay(engine: Engine, lines: Iterable[str], out_dir: str, out: TextIO = sys.stdout) -> int:
    """Runs every step of the trace; returns the number of steps."""
    os.makedirs(out_dir, exist_ok=True)
    slots: Dict[str, int] = {}
    n = 0
    for raw in lines:
        raw = raw.strip()
        if not raw:
            continue
        try:
            rec = json.loads(raw)
        except json.JSONDecodeError as e:
            raise TraceError(f"trace line {n + 1} is not JSON: {e}") from e
        step = rec.get("step", n)
        entries = rec.get("entries", [])
        batch, want = [], []
        for ent in entries:
            rid = str(ent["id"])
            if rid not in slots:
                slots[rid] = engine.alloc_slot()
            batch.append((slots[rid], ent["tokens"]))
            want.append(ent.get("want", []))
        if batch:
            logits = engine.step(batch, want=want)
            if logits is not None:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid not in slots:
                raise TraceError(f"step {step} ends request '{rid}', which is not live")
            engine.free_slot(slots.pop(rid))
        print(f"done {step}", file=out, flush=True)
        n += 1
    return n


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description="replay token traces through the engine and write logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64); sizes the cache")
    args = ap.parse_args(argv)
    engine = Engine.from_folder(args.model, dtype=args.dtype, max_tokens=args.max_tokens)
    replay(engine, sys.stdin, args.out)
    return 0
