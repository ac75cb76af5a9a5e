"""Command line in the manner of the reference's (Daisi.Llogos.Cli/Program.cs:444-576):
the same option names, meanings and defaults where it has them.  Prompts are token ids
(the tokenizer is not part of this library); text is accepted when the model folder has a
tokenizer.json and the `tokenizers` package is importable."""
from __future__ import annotations

import os
import sys
import time

USAGE = """daisi-llogos_amd - dense-decoder inference on one AMD MI355X

Usage: python -m daisi-llogos_amd --model <folder> --prompt <token ids> [options]

Options:
  --model, -m <path>       Model folder with config.json and model.safetensors (required)
  --prompt, -p <ids>       Prompt as token ids ("1 2 3" or "1,2,3" or @file); several prompts
                           separated by ';' run as one batch (required unless --bench)
  --max-tokens, -n <n>     Maximum tokens to generate (default: 256)
  --max-context <n>        Maximum context length (default: 2048)
  --temperature, -t <f>    Sampling temperature, 0=greedy (default: 0.7)
  --top-k <n>              Top-k sampling, 0=disabled (default: 40)
  --top-p <f>              Top-p nucleus sampling (default: 0.9)
  --repeat-penalty <f>     Repetition penalty (default: 1.1)
  --seed <n>               Random seed for reproducibility
  --backend, -b <name>     Compute backend: hip (the only one)
  --bench                  Run benchmark (prefill + decode timing)
  --attention <mode>       Attention strategy: full, window:<N>, sinks:<S>,<W> (default: full)
  --dtype <name>           bfloat16 (default) or float32
  --batch <n>              Sequences generated together (default: number of prompts; bench: 1)
  --prompt-len <n>         Bench without --prompt: random prompt of this length (default: 512)
  --help, -h               Show this help

Random weights (a model folder from a configuration and a seed):
  python -m daisi-llogos_amd random --config <config.json> --output-dir <folder> [--seed <n>]
"""


class CliArgs:
    def __init__(self):
        self.model = None
        self.prompt = None
        self.max_tokens = 256
        self.max_context = 2048
        self.temperature = 0.7
        self.top_k = 40
        self.top_p = 0.9
        self.repeat_penalty = 1.1
        self.seed = None
        self.backend = "hip"
        self.bench = False
        self.attention = "full"
        self.dtype = "bfloat16"
        self.batch = None
        self.prompt_len = 512
        self.help = False


def parse_args(argv) -> CliArgs:
    a = CliArgs()
    i = 0

    def nxt():
        nonlocal i
        i += 1
        if i >= len(argv):
            raise ValueError(f"Missing value for {argv[i - 1]}")
        return argv[i]
    while i < len(argv):
        o = argv[i]
        if o in ("--model", "-m"): a.model = nxt()
        elif o in ("--prompt", "-p"): a.prompt = nxt()
        elif o in ("--max-tokens", "-n"): a.max_tokens = int(nxt())
        elif o == "--max-context": a.max_context = int(nxt())
        elif o in ("--temperature", "-t"): a.temperature = float(nxt())
        elif o == "--top-k": a.top_k = int(nxt())
        elif o == "--top-p": a.top_p = float(nxt())
        elif o == "--repeat-penalty": a.repeat_penalty = float(nxt())
        elif o == "--seed": a.seed = int(nxt())
        elif o in ("--backend", "-b"): a.backend = nxt()
        elif o == "--bench": a.bench = True
        elif o == "--attention": a.attention = nxt()
        elif o == "--dtype": a.dtype = nxt()
        elif o == "--batch": a.batch = int(nxt())
        elif o == "--prompt-len": a.prompt_len = int(nxt())
        elif o in ("--help", "-h"): a.help = True
        else:
            raise ValueError(f"unknown option {o}")
        i += 1
    return a


def parse_prompts(text: str, model_dir: str):
    if text.startswith("@"):
        with open(text[1:]) as fh:
            text = fh.read()
    prompts = []
    for part in text.split(";"):
        part = part.strip()
        if not part:
            continue
        fields = part.replace(",", " ").split()
        if all(f.lstrip("-").isdigit() for f in fields):
            prompts.append([int(f) for f in fields])
            continue
        tok_file = os.path.join(model_dir, "tokenizer.json")
        if not os.path.isfile(tok_file):
            raise ValueError("the prompt is not a list of token ids and the model folder has no tokenizer.json")
        from tokenizers import Tokenizer
        prompts.append(Tokenizer.from_file(tok_file).encode(part).ids)
    if not prompts:
        raise ValueError("empty prompt")
    return prompts


def run_random(argv) -> int:
    """`random --config FILE --output-dir DIR [--seed N]`: config.json + model.safetensors with
    random weights for the configuration's architecture (the reference has no such mode; its
    sub-commands are `split` and `train`, Daisi.Llogos.Cli/Program.cs:25-31)."""
    import json
    config = out = None
    seed = 0
    i = 0
    try:
        while i < len(argv):
            if argv[i] == "--config": config = argv[i + 1]; i += 1
            elif argv[i] in ("--output-dir", "-o"): out = argv[i + 1]; i += 1
            elif argv[i] == "--seed": seed = int(argv[i + 1]); i += 1
            else:
                raise ValueError(f"unknown option {argv[i]}")
            i += 1
    except (IndexError, ValueError) as e:
        print(f"Error: {e if isinstance(e, ValueError) else 'missing value'}", file=sys.stderr)
        return 1
    if not config or not out:
        print("Error: random needs --config and --output-dir", file=sys.stderr)
        return 1
    if not os.path.isfile(config):
        print(f"Error: configuration not found: {config}", file=sys.stderr)
        return 1
    from .weights.random_init import write_random_model
    with open(config) as fh:
        data = json.load(fh)
    write_random_model(out, data, seed=seed)
    print(f"wrote {out}/config.json and {out}/model.safetensors (seed {seed})", file=sys.stderr)
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "random":
        return run_random(argv[1:])
    try:
        args = parse_args(argv)
    except ValueError as e:
        print(f"Error: {e}", file=sys.stderr)
        return 1
    if args.help or not argv:
        print(USAGE, file=sys.stderr)
        return 0
    if not args.model:
        print("Error: --model is required", file=sys.stderr)
        return 1
    if not os.path.isdir(args.model):
        print(f"Error: model folder not found: {args.model}", file=sys.stderr)
        return 1
    if not args.bench and not args.prompt:
        print("Error: --prompt is required", file=sys.stderr)
        return 1
    if args.backend.lower() not in ("hip", "rocm", "gpu"):
        print(f"Error: backend '{args.backend}' is not available; this library runs on HIP only", file=sys.stderr)
        return 1

    import numpy as np
    from .api import Llogos
    from .sampling.params import GenerationParams

    t0 = time.perf_counter()
    if args.prompt:
        prompts = parse_prompts(args.prompt, args.model)
    else:
        prompts = None
    n_batch = args.batch or (len(prompts) if prompts else 1)
    llm = Llogos(args.model, dtype=args.dtype, max_context=args.max_context, max_batch=n_batch,
                 attention=args.attention)
    load_ms = (time.perf_counter() - t0) * 1000
    model = llm.engine.model
    print(f"Loaded {llm.engine.architecture}: {model.describe()} in {load_ms:.0f} ms", file=sys.stderr)

    if args.bench:
        if prompts is None:
            rng = np.random.default_rng(args.seed or 0)
            prompts = [rng.integers(0, model.spec.vocab_size, size=args.prompt_len).tolist() for _ in range(n_batch)]
        print(f"Benchmarking with {len(prompts)} prompt(s) of {len(prompts[0])} tokens", file=sys.stderr)
        print(f"Backend: hip ({args.dtype}), Max tokens: {args.max_tokens}\n", file=sys.stderr)
        r = llm.benchmark(prompts, args.max_tokens)
        total_ms = (r.prefill_seconds + r.decode_seconds) * 1000
        print("=== Benchmark Results ===", file=sys.stderr)
        print(f"  Prefill:  {r.prompt_tokens:6d} tokens in {r.prefill_seconds * 1000:8.1f} ms  "
              f"({r.prefill_tokens_per_second:8.1f} tok/s)", file=sys.stderr)
        print(f"  Decode:   {r.generated_tokens:6d} tokens in {r.decode_seconds * 1000:8.1f} ms  "
              f"({r.decode_tokens_per_second:8.1f} tok/s)", file=sys.stderr)
        print(f"  Total:    {r.prompt_tokens + r.generated_tokens:6d} tokens in {total_ms:8.1f} ms", file=sys.stderr)
        print(f"  Load:     {load_ms:8.1f} ms", file=sys.stderr)
        # against the GPU's published peaks: the prompt step's flops, and the bytes the decode steps had to read
        hbm = (r.peaks or {}).get("hbm", 0.0)
        print(f"  Roofline: prefill {r.prefill_flops / max(r.prefill_seconds, 1e-12) / 1e12:7.1f} TFLOP/s "
              f"({r.prefill_fraction_of_peak:.3f} of the {r.dtype} matrix peak)  "
              f"decode {r.decode_bytes_per_second / 1e9:7.1f} GB/s "
              + (f"({r.decode_fraction_of_peak:.3f} of {hbm / 1e12:g} TB/s)" if hbm else "(no published peak for this GPU)"),
              file=sys.stderr)
        print(f"  Memory:   weights {model.step_weight_bytes() / 1e9:.2f} GB, packed copies "
              f"{model.packed_weight_bytes() / 1e9:.2f} GB, cache {llm.engine.cache.bytes() / 1e9:.2f} GB", file=sys.stderr)
        return 0

    params = GenerationParams(max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k,
                              top_p=args.top_p, repetition_penalty=args.repeat_penalty, seed=args.seed)
    single = len(prompts) == 1

    def on_token(request: int, token: int) -> None:
        if single:
            print(token, end=" ", flush=True)
    res = llm.generate(prompts, params, on_token=on_token)
    if single:
        print()
    else:
        for toks in res.tokens:
            print(" ".join(str(t) for t in toks))
    print(f"\n[prefill: {res.prompt_tokens} tokens, {res.prefill_tokens_per_second:.1f} tok/s | "
          f"decode: {res.generated_tokens} tokens, {res.decode_tokens_per_second:.1f} tok/s]", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
