"""Decode and prefill throughput of the Llama-3.1-8B layer sizes with random bfloat16
weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--prompt-len P] [--model NAME]

A step is one decode step of the whole batch.  The line printed at the end is the record:
value = decoded tokens a second at the default batch of 8 (512-token random prompts, the
context grows from there), "prefill" = one 2,048-token prompt, "roofline" = bytes the decode
step has to read (every weight it uses once, the cache of the live requests) / its time
against 8 TB/s, "points" = decoding at batch 1 and 64.  Beside the published peaks the record
holds what this GPU was measured to do at best in the same run ("measured_peak": a kernel that
only reads the weights' bytes; v_mfma_f32_16x16x32_bf16 issued back to back) and the fractions
of those; "generate_loop" is the same decode through the product's generation loop
(Generator.generate: its batching, stop checks and bookkeeping inside the timed region);
"spread" = the headline decode measured three times; "kernels" = where a decode step at the
headline batch and the 2,048-token prompt spend their time, part by part, from events on the
stream (microseconds a call, GB/s of the bytes a part has to read or TFLOP/s of its products);
"sizes" = decoding at further sizes and contexts (the same model at 16,384 positions and at
batch 64 with 4,096 positions; the Qwen3-14B layer sizes at batch 8 and 32), each with its
fraction of the memory roofline.

    python bench.py --ceilings      # the measured ceilings alone, at several buffer sizes"""
import argparse
import importlib
import json
import sys
import time

HBM_PEAK = 8.0e12            # bytes/s, MI355X
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense flop/s

LLAMA31_8B = {
    "architectures": ["LlamaForCausalLM"], "vocab_size": 128256, "hidden_size": 4096, "intermediate_size": 14336,
    "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "max_position_embeddings": 131072,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "attention_bias": False, "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 128001,
}
QWEN3_14B = {
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 151936, "hidden_size": 5120, "intermediate_size": 17408,
    "num_hidden_layers": 40, "num_attention_heads": 40, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "max_position_embeddings": 40960,
    "attention_bias": False, "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 151645,
}
LLAMA31_70B = dict(LLAMA31_8B, hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64)
# the size class of the reference's own published runs (Llama-3.2-1B: head size 64, tied head)
LLAMA32_1B = dict(LLAMA31_8B, hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, head_dim=64,
                  tie_word_embeddings=True,
                  rope_scaling=dict(LLAMA31_8B["rope_scaling"], factor=32.0))
MODELS = {"llama-3.1-8b": ("Llama-3.1-8B", LLAMA31_8B), "qwen3-14b": ("Qwen3-14B", QWEN3_14B),
          "llama-3.1-70b": ("Llama-3.1-70B", LLAMA31_70B), "llama-3.2-1b": ("Llama-3.2-1B", LLAMA32_1B)}
CONTEXT, PROMPT, PREFILL_TOKENS = 4096, 512, 2048


def weight_bytes(cfg, elt=2):
    """Bytes of every matrix a decode step reads once: the layers' projections and the head
    (the embedding table is read for a few rows only)."""
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    q = cfg["num_attention_heads"] * cfg["head_dim"]
    kv = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = h * (q + 2 * kv) + q * h + 3 * h * i + 2 * h        # + the two norm weights
    return (cfg["num_hidden_layers"] * per_layer + v * h + h) * elt


def kv_bytes_per_token(cfg, elt=2):
    return cfg["num_hidden_layers"] * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * elt


def prefill_flops(cfg, t):
    """2 * (matrix parameters) per token, causal attention 2 * 2 * heads * head_dim * t^2 / 2 per
    layer, the head on one row."""
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    q = cfg["num_attention_heads"] * cfg["head_dim"]
    kv = cfg["num_key_value_heads"] * cfg["head_dim"]
    linear = cfg["num_hidden_layers"] * (h * (q + 2 * kv) + q * h + 3 * h * i)
    attn = cfg["num_hidden_layers"] * 2 * q * t * t                  # qk^T and pv, half of the square each
    return 2 * linear * t + attn + 2 * v * h


def clocks_under_load(torch, K, seconds=3.0):
    """The GPU's clock (rocm-smi, read from a thread) while one kind of work runs in a loop: idle, a few-row product
    that waits for memory, MFMAs on registers, and the gate/up product of 2,048 rows of the 8B sizes by the tiled
    kernel and by the library.  The prompt's products run against the power limit: the clock says how far."""
    import re
    import shutil
    import subprocess
    import threading
    import time
    if shutil.which("rocm-smi") is None:
        print("[ceilings] clocks: no rocm-smi on this machine", flush=True)
        return
    dev = "cuda:0"

    def sample(stop, out):
        while not stop.is_set():
            try:
                text = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=10).stdout
                m = re.search(r"sclk clock level[^\n]*\((\d+)Mhz\)", text)
                if m:
                    out.append(int(m.group(1)))
            except (OSError, subprocess.SubprocessError):
                return
            time.sleep(0.2)

    def under(label, fn, flops=0.0):
        stop, seen = threading.Event(), []
        th = threading.Thread(target=sample, args=(stop, seen))
        th.start()
        t0, n = time.time(), 0
        while time.time() - t0 < seconds:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            n += 20
        dt = (time.time() - t0) / n
        stop.set()
        th.join()
        mhz = sorted(seen[1:])[len(seen[1:]) // 2] if len(seen) > 1 else 0
        rate = f", {flops / dt / 1e15:.3f} PFLOP/s, {flops / dt / (MFMA_PEAK['bf16'] * mhz / 2400.0) :.2f} of the peak at that clock" if flops and mhz else ""
        print(f"[ceilings] clock under {label}: {mhz} MHz ({dt * 1e6:.0f} us a call{rate})", flush=True)

    M, I, H = 2048, 14336, 4096
    a = (torch.randn(M, H, device=dev) * 0.5).to(torch.bfloat16)
    w = (torch.randn(2 * I, H, device=dev) * 0.02).to(torch.bfloat16)
    pw = K.pack_weights(w, I)
    wd = [K.pack_weights((torch.randn(H, I, device=dev) * 0.02).to(torch.bfloat16)) for _ in range(8)]
    a8 = torch.randn(8, I, device=dev).to(torch.bfloat16)
    turn = [0]

    def few_rows():
        turn[0] = (turn[0] + 1) % len(wd)
        K.gemm_packed_bf16(a8, wd[turn[0]], None, torch.float32, 8, 128)
    time.sleep(1.0)
    under("nothing", lambda: None)
    under("the down product of 8 rows (memory-bound)", few_rows)
    under("MFMAs on registers", lambda: K.measure_mfma_rate(iters=2000, shapes=(32,)))
    flops = 2.0 * M * 2 * I * H
    under("the tiled gate/up product of 2,048 rows", lambda: K.gemm_tiles_bf16(a, pw, None, torch.bfloat16), flops)
    under("the library's gate/up product of 2,048 rows", lambda: torch.matmul(a, w.t()), flops)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=248)   # + 8 warm-up = 256 new tokens
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--model", choices=sorted(MODELS), default="llama-3.1-8b", help="whose layer sizes to run")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="tokens of each sequence's prompt before decoding")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="tokens of the timed prompt")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has (0 = all)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--no-sizes", action="store_true", help="skip the further sizes and contexts")
    ap.add_argument("--only-prefill", action="store_true", help="time the 2,048-token prompt alone (for profiling)")
    ap.add_argument("--ceilings", action="store_true", help="measure the read bandwidth and the MFMA rate of this GPU and exit")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy (the default run); above 0 the sampler draws")
    ap.add_argument("--top-k", type=int, default=40)
    ap.add_argument("--top-p", type=float, default=0.9)
    args = ap.parse_args(argv)
    prefill_tokens = args.prefill_tokens
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2

    import numpy as np
    import torch
    llogos = importlib.import_module("daisi-llogos_amd")
    K = importlib.import_module("daisi-llogos_amd.ops.kernels")
    fetch_tokens = importlib.import_module("daisi-llogos_amd.engine.generate").fetch_tokens

    if args.ceilings:
        # the sizes are those of the 8B matrices a decode step streams: gate/up, down, qkv, o, and all weights of a layer
        for label, n in (("gate/up 235 MB", 2 * 14336 * 4096 * 2), ("down 117 MB", 4096 * 14336 * 2), ("qkv 50 MB", 6144 * 4096 * 2),
                         ("o 34 MB", 4096 * 4096 * 2), ("1 GiB", 1 << 30), ("4 GiB", 1 << 32)):
            bw = K.measure_read_bandwidth(n)
            print(f"[ceilings] read {label}: {bw / 1e12:.2f} TB/s ({bw / HBM_PEAK:.3f} of {HBM_PEAK / 1e12:g})", flush=True)
        for shape in (16, 32):
            for noisy in (False, True):
                rate = K.measure_mfma_rate(shapes=(shape,), noisy=noisy)
                print(f"[ceilings] mfma bf16 {'16x16x32' if shape == 16 else '32x32x16'}, "
                      f"{'random operands' if noisy else 'constant operands'}: {rate / 1e15:.3f} PFLOP/s "
                      f"({rate / MFMA_PEAK['bf16']:.3f} of {MFMA_PEAK['bf16'] / 1e15:g})", flush=True)
        clocks_under_load(torch, K)
        return 0

    model_name, cfg = MODELS[args.model]
    cfg = dict(cfg)
    cfg0 = cfg
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    max_batch = max(args.batch, 1 if (args.no_points or args.only_prefill) else 64)
    per_seq = args.prompt_len + args.steps + args.warmup + 64
    sizes_on = not (args.no_points or args.only_prefill or args.no_sizes or args.temperature > 0)
    long_runs = [(8, 16384), (64, 4096)] if sizes_on else []        # (batch, positions) of the same model
    t0 = time.time()
    eng = eng0 = llogos.Engine.from_config(cfg, seed=0, dtype="bfloat16",
                                    max_tokens=max([max_batch * (per_seq + 64), prefill_tokens + 128] +
                                                   [b * (n + 64) for b, n in long_runs]), n_slots=max_batch)
    print(f"[bench] model ready in {time.time() - t0:.1f} s; weights {weight_bytes(cfg) / 1e9:.2f} GB, "
          f"cache {eng.cache.bytes() / 1e9:.2f} GB", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    if args.temperature > 0:
        S = importlib.import_module("daisi-llogos_amd.sampling")
        sampler = S.Sampler(S.GenerationParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                                               repetition_penalty=1.0, seed=0))
        sampling = f"temperature {args.temperature:g}, top-k {args.top_k}, top-p {args.top_p:g}"
    else:
        sampler, sampling = None, "greedy"

    def pick(logits, step):
        """The step's tokens on the device: the first maximum, or the sampler's draw."""
        if sampler is None:
            return K.argmax(logits)
        n = logits.shape[0]
        return sampler.sample(logits, list(range(n)), [step] * n, None)

    def decode_run(batch, steps, warmup, eng=None, cfg=None, prompt_len=None, prompts_per_step=None):
        """Prompts in one step (or `prompts_per_step` at a time), then greedy single-token steps:
        `warmup` untimed, `steps` timed."""
        eng, cfg, prompt_len = eng or eng0, cfg or cfg0, prompt_len or args.prompt_len
        slots = [eng.alloc_slot() for _ in range(batch)]
        prompts = [rng.integers(0, cfg["vocab_size"], size=prompt_len).tolist() for _ in range(batch)]
        per = prompts_per_step or batch
        logits = torch.cat([eng.step(list(zip(slots[i:i + per], prompts[i:i + per])), want="last") for i in range(0, batch, per)])
        ids = pick(logits, 0)
        rows = list(range(batch))
        placeholders = [(s, [0]) for s in slots]
        done = [0]

        def run(n):
            """Greedy single-token steps as the generation loop runs them: a step takes its
            tokens from the device memory the last argmax wrote, and the host reads the last
            step's tokens while this one runs."""
            nonlocal ids
            for _ in range(n):
                tokens = fetch_tokens(ids)
                logits = eng.step(placeholders, want="last", device_ids=(ids, rows), borrow=True)
                done[0] += 1
                ids = pick(logits, done[0])
                tokens()
        run(warmup)
        torch.cuda.synchronize()
        t = time.perf_counter()
        run(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_mid = prompt_len + warmup + steps / 2.0
        for s in slots:
            eng.free_slot(s)
        return dt, ctx_mid

    def bytes_of_step(cfg, batch, ctx_mid):
        """What a decode step has to read: every weight it uses once, and the cache of the live requests."""
        return weight_bytes(cfg) + batch * ctx_mid * kv_bytes_per_token(cfg)

    def part_costs(cfg, tokens, batch, context):
        """Per part of a layer: bytes of its weights (and of the cache it reads), flops of `tokens` tokens."""
        h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
        q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
        mats = {"qkv": h * (q + 2 * kv), "o": q * h, "gate_up": 2 * h * i, "down": h * i, "head": v * h}
        costs = {k: (2.0 * n, 2.0 * n * (batch if k == "head" else tokens)) for k, n in mats.items()}
        # attention: keys and values of the live context; products with keys and values over the causal half
        pairs = batch * context if tokens == batch else tokens * (tokens + 1) / 2.0
        costs["attention"] = (batch * context * 2.0 * kv * 2, 4.0 * q * pairs)
        return costs

    def prompt_rates(eng, cfg, entries, tokens):
        """A prompt step launched kernel by kernel with a probe: per part microseconds a call and TFLOP/s."""
        probe = llogos.StepProbe()
        probe.hold()
        probe.start()
        eng.step(entries, want="last", probe=probe)
        us = probe.microseconds_per_call()
        out = {}
        for name, (_, flops) in part_costs(cfg, tokens, 1, tokens).items():
            if name in us:
                out[name + "_us"] = round(us[name], 1)
                out[name + "_TFLOPs"] = round(flops / us[name] / 1e6, 1)
        for name in ("norm", "rotation"):
            if name in us:
                out[name + "_us"] = round(us[name], 1)
        return out

    def decode_rates(eng, cfg, slots, context, step_us):
        """The parts of a single-token step of the sequences in `slots`: the products and the norm each run
        for every layer in a row (the weights come from memory, nothing lies between the kernels, as in the
        replayed step): microseconds a call and GB/s of the bytes the part has to read.  The attention
        (rotation, cache write, attention, merge) is what is left of the replayed step (`step_us`, less the
        head) per layer beside those; launched kernel by kernel its four short kernels would be measured
        with the gaps between them, and a record between every two kernels costs them more than they take."""
        batch = len(slots)
        probe = llogos.StepProbe()
        eng.step([(sl, [1]) for sl in slots], want="last", probe=probe)     # (gives the step's context to the probe)
        layers = eng.model.layers
        dev = eng.rt.device
        h = torch.randn(batch, cfg["hidden_size"], device=dev).to(torch.bfloat16)
        a = torch.randn(batch, cfg["num_attention_heads"] * cfg["head_dim"], device=dev).to(torch.bfloat16)
        act = torch.randn(batch, cfg["intermediate_size"], device=dev).to(torch.bfloat16)

        def gate_up(layer, rows):
            out = layer.ffn.gate_up.gated_product(rows)
            return out if out is not None else layer.ffn.gate_up.product(rows)
        P = llogos.parts
        x = torch.randn(batch, cfg["hidden_size"], device=dev)
        # steps of few rows: o and down add themselves to the stream where their shapes allow and leave the next
        # norm's rows, which gate/up and qkv take as they are (no norm kernel between); otherwise products in
        # parts and the norm's kernel
        def closing(product, act, norm):
            if product.add_to(act, P.Residual(x, norm)) is not None:
                return (lambda: product.add_to(act, P.Residual(x, norm))), norm.forward(x, product.add_to(act, P.Residual(x, norm)), lazy=True)
            return (lambda: product.product(act, f32_ok=True)), h
        o_calls, rows_ffn = zip(*[closing(l.mixer.o, a, l.ffn_norm) for l in layers])
        down_calls, rows_mixer = zip(*[closing(l.ffn.down, act, l.mixer_norm) for l in layers])
        norms_a_layer = sum(1 for r in (rows_ffn[0], rows_mixer[0]) if r is h)
        us = {
            "qkv": probe.repeat([lambda l=l, r=r: l.mixer.qkv.product(r, f32_ok=True) for l, r in zip(layers, rows_mixer)]),
            "o": probe.repeat(list(o_calls)),
            "gate_up": probe.repeat([lambda l=l, r=r: gate_up(l, r) for l, r in zip(layers, rows_ffn)]),
            "down": probe.repeat(list(down_calls)),
            "norm": probe.repeat([lambda l=l: l.mixer_norm.forward(torch.zeros(batch, cfg["hidden_size"], device=dev), None)
                                  for l in layers]) if norms_a_layer else 0.0,
        }
        us["head"] = probe.repeat([lambda: eng.model.head.forward(h, out_dtype=torch.float32)] * 3)
        us["attention"] = (step_us - us["head"]) / len(layers) - us["qkv"] - us["o"] - us["gate_up"] - us["down"] - norms_a_layer * us["norm"]
        out = {}
        for name, (nbytes, _) in part_costs(cfg, batch, batch, context).items():
            out[name + "_us"] = round(us[name], 1)
            out[name + "_GBps"] = round(nbytes / us[name] / 1e3, 1)
        out["norm_us"] = round(us["norm"], 1)
        return out

    if args.only_prefill:
        prompt = rng.integers(0, cfg["vocab_size"], size=prefill_tokens).tolist()
        for it in range(4):
            s = eng.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            eng.step([(s, prompt)], want="last")
            torch.cuda.synchronize()
            print(f"[bench] prefill {prefill_tokens} tokens, {cfg['num_hidden_layers']} layers: "
                  f"{(time.perf_counter() - t) * 1e3:.2f} ms", file=sys.stderr, flush=True)
            eng.free_slot(s)
        return 0

    dt, ctx_mid = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes(cfg) + args.batch * ctx_mid * kv_bytes_per_token(cfg)
    achieved = step_bytes / (dt / args.steps)
    record = {
        "metric": f"decode tok/s, {model_name} bf16", "value": round(value, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": f"{model_name} sizes, random weights", "global_batch": args.batch, "seq_len": CONTEXT,
                   "parallelism": "single GPU", "prompt_len": args.prompt_len, "layers": cfg["num_hidden_layers"],
                   "layers_full": full_layers, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "rope_theta": cfg["rope_theta"], "rope_scaling": f"llama3 x{cfg['rope_scaling']['factor']:g}" if cfg.get("rope_scaling") else "none", "rms_eps": cfg["rms_norm_eps"],
                   "sampling": sampling, "hip_graphs": eng.graphs is not None},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {ms_per_step:.3f} ms/step, "
          f"{achieved / 1e12:.2f} TB/s", file=sys.stderr, flush=True)

    if not args.no_points:
        runs = [value] + [args.batch * args.steps / decode_run(args.batch, args.steps, args.warmup)[0] for _ in range(2)]
        record["spread"] = {"runs": 3, "min": round(min(runs), 1), "max": round(max(runs), 1)}
        print(f"[bench] decode b{args.batch}, three runs: {min(runs):.1f} to {max(runs):.1f} tok/s", file=sys.stderr, flush=True)
    if not args.no_points and sampler is None:
        # the same decode through the product's own loop: prompts in one step, then greedy tokens with
        # the loop's batching, stop checks, slot bookkeeping and token fetches inside the timed region
        S = importlib.import_module("daisi-llogos_amd.sampling")
        generator = llogos.Generator(eng, max_batch=args.batch, synchronize=torch.cuda.synchronize)
        prompts = [rng.integers(0, cfg["vocab_size"], size=args.prompt_len).tolist() for _ in range(args.batch)]
        n_new = args.steps + args.warmup
        res = generator.generate(prompts, S.GenerationParams.greedy(max_tokens=n_new, stop_tokens=()))
        loop_steps = n_new - 1                                   # the first token comes from the prompt step
        record["generate_loop"] = {"value": round(args.batch * loop_steps / res.decode_seconds, 1), "unit": "tok/s",
                                   "ms_per_step": round(res.decode_seconds / loop_steps * 1e3, 4), "steps": loop_steps}
        print(f"[bench] generation loop b{args.batch}: {record['generate_loop']['value']:.1f} tok/s, "
              f"{record['generate_loop']['ms_per_step']:.3f} ms/step", file=sys.stderr, flush=True)
    if not args.no_points:
        points, fractions = {}, {}
        for b in (1, 64):
            steps = args.steps
            d, mid = decode_run(b, steps, args.warmup)
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            # the same account as for the headline step: every weight once and the live requests' cache
            fractions[f"decode_b{b}"] = round((weight_bytes(cfg) + b * mid * kv_bytes_per_token(cfg)) / (d / steps) / HBM_PEAK, 4)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']:.1f} tok/s, {d / steps * 1e3:.3f} ms/step, "
                  f"{fractions[f'decode_b{b}']:.3f} of {HBM_PEAK / 1e12:g} TB/s", file=sys.stderr, flush=True)
        record["points"] = points
        record["points_roofline_frac"] = fractions
    if not args.no_points:
        prompt = rng.integers(0, cfg["vocab_size"], size=prefill_tokens).tolist()
        times = []
        for it in range(5):                              # the first warms the library up; the best of the rest counts
            s = eng.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            eng.step([(s, prompt)], want="last")
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            eng.free_slot(s)
        pt = min(times[1:])
        flops = prefill_flops(cfg, prefill_tokens)
        record["prefill"] = {"value": round(prefill_tokens / pt, 1), "tokens": prefill_tokens, "ms": round(pt * 1e3, 3),
                             "frac": round(flops / pt / MFMA_PEAK["bf16"], 4)}
        print(f"[bench] prefill {prefill_tokens}: {prefill_tokens / pt:.0f} tok/s, {pt * 1e3:.2f} ms (five runs: "
              f"{min(times) * 1e3:.2f} to {max(times[1:]) * 1e3:.2f} after the first)", file=sys.stderr, flush=True)
        record["prefill"]["ms_max"] = round(max(times[1:]) * 1e3, 3)
    # What this GPU does at best: reading as many bytes as the model's weights, and the matrix cores' issue rate.
    # (After the timed decode steps and prompts: seconds of MFMAs at the power limit just before them cost the
    # decode steps 2 %.)
    read_peak = K.measure_read_bandwidth(min(weight_bytes(cfg), 4 << 30), repeats=5)
    mfma_peak = K.measure_mfma_rate()
    print(f"[bench] measured ceilings: read {read_peak / 1e12:.2f} TB/s, mfma bf16 {mfma_peak / 1e15:.3f} PFLOP/s",
          file=sys.stderr, flush=True)
    record["roofline"].update(measured_peak=round(read_peak / 1e9, 1), frac_of_measured=round(achieved / read_peak, 4))
    if not args.no_points:
        record["prefill"].update(measured_peak_tflops=round(mfma_peak / 1e12, 1),
                                 frac_of_measured=round(prefill_flops(cfg, prefill_tokens) / pt / mfma_peak, 4))
        # where the time goes: a decode step of the headline batch and the prompt, part by part
        slots = [eng.alloc_slot() for _ in range(args.batch)]
        eng.step([(sl, rng.integers(0, cfg["vocab_size"], size=args.prompt_len).tolist()) for sl in slots], want="last")
        kernels = {f"decode_b{args.batch}": decode_rates(eng, cfg, slots, args.prompt_len + 1, ms_per_step * 1e3)}
        for sl in slots:
            eng.free_slot(sl)
        s = eng.alloc_slot()
        kernels[f"prefill_{prefill_tokens}"] = prompt_rates(eng, cfg, [(s, prompt)], prefill_tokens)
        eng.free_slot(s)
        record["kernels"] = kernels
        for k, v in kernels.items():
            print(f"[bench] {k}: {v}", file=sys.stderr, flush=True)
    if sizes_on:
        sizes = {}

        def size_point(label, eng, cfg, batch, prompt_len, steps, per_step):
            d, mid = decode_run(batch, steps, 4, eng=eng, cfg=cfg, prompt_len=prompt_len, prompts_per_step=per_step)
            frac = bytes_of_step(cfg, batch, mid) / (d / steps) / HBM_PEAK
            sizes[label] = {"value": round(batch * steps / d, 1), "ms_per_step": round(d / steps * 1e3, 3), "frac": round(frac, 4)}
            print(f"[bench] {label}: {sizes[label]['value']:.1f} tok/s, {d / steps * 1e3:.3f} ms/step, {frac:.3f} of "
                  f"{HBM_PEAK / 1e12:g} TB/s", file=sys.stderr, flush=True)

        short = model_name.lower().replace("-", "").replace(".", "")
        for b, n in long_runs:                               # the context is n positions in the middle of the timed steps
            size_point(f"{short}_b{b}_ctx{n}", eng, cfg, b, n - 4 - 16, 32, max(1, 32768 // n))
        if args.model == "llama-3.1-8b" and not args.layers:
            # another model's sizes: the engine above gives its memory back first
            del eng, eng0, generator
            import gc
            gc.collect()
            torch.cuda.empty_cache()
            name2, cfg2 = MODELS["qwen3-14b"]
            t0 = time.time()
            eng2 = llogos.Engine.from_config(dict(cfg2), seed=0, dtype="bfloat16", max_tokens=32 * (1024 + 128 + 64), n_slots=32)
            print(f"[bench] {name2} ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
            for b in (8, 32):
                size_point(f"qwen314b_b{b}_p1024", eng2, cfg2, b, 1024, 64, 8)
        record["sizes"] = sizes
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
