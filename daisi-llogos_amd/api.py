"""The Python entry point: load a model folder, generate, benchmark.

The reference's entry points are TextGenerator.Generate / Benchmark
(Daisi.Llogos/Inference/TextGenerator.cs:26-186) behind its command line
(Daisi.Llogos.Cli/Program.cs); option names and defaults follow them."""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple, Union

import torch

from .cache.pages import PAGE_TOKENS, pages_for
from .engine.generate import GenerationResult, Generator
from .engine.step import Engine
from .sampling.params import GenerationParams


def parse_attention(value: str) -> Tuple[Optional[int], int]:
    """'full', 'window:N' or 'sinks:S,W' (Daisi.Llogos/Inference/AttentionStrategy.cs:75-100)
    -> (window or None for the configuration's own, sinks)."""
    v = value.strip().lower()
    if v == "full":
        return None, 0
    if v.startswith("window:"):
        n = int(v[7:])
        if n <= 0:
            raise ValueError("window size must be positive")
        return n, 0
    if v.startswith("sinks:"):
        parts = v[6:].split(",")
        if len(parts) != 2:
            raise ValueError("sinks format: sinks:<sink_tokens>,<window_size>")
        s, w = int(parts[0]), int(parts[1])
        if s < 0 or w <= 0:
            raise ValueError("sinks needs sink_tokens >= 0 and window_size > 0")
        return s + w, s
    raise ValueError(f"unknown attention strategy: {value}. Use full, window:<N>, or sinks:<S>,<W>")


@dataclass
class BenchmarkResult:
    """As the reference's BenchmarkResult (TextGenerator.cs:238-247), summed over the batch."""
    prompt_tokens: int
    generated_tokens: int
    prefill_seconds: float
    decode_seconds: float

    @property
    def prefill_tokens_per_second(self) -> float:
        return self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_tokens_per_second(self) -> float:
        return self.generated_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0


class Llogos:
    """A loaded model that generates.

        llm = Llogos("/path/to/model", dtype="bfloat16", max_context=2048, max_batch=8)
        out = llm.generate([[1, 2, 3], [4, 5]], max_tokens=16, temperature=0)
        out.tokens  ->  [[...], [...]]
    """

    def __init__(self, model: str, dtype: Union[str, torch.dtype] = "bfloat16", max_context: int = 2048,
                 max_batch: int = 8, max_tokens_in_cache: Optional[int] = None, attention: str = "full",
                 device: str = "cuda:0"):
        window, sinks = parse_attention(attention)
        options = {}
        if window is not None:
            options = dict(attention_window=window - sinks, attention_sinks=sinks)
        pool = max_tokens_in_cache or max_batch * pages_for(max_context) * PAGE_TOKENS
        self.max_context, self.max_batch = max_context, max_batch
        self.engine = Engine.from_folder(model, dtype=dtype, max_tokens=pool, n_slots=max(max_batch, 1),
                                         device=device, **options)
        self.config = self.engine.config
        self._generator = Generator(self.engine, max_batch=max_batch, synchronize=torch.cuda.synchronize)

    def generate(self, prompts: Sequence[Sequence[int]], params: Optional[GenerationParams] = None,
                 on_token=None, **options) -> GenerationResult:
        """prompts: token id lists (one list is taken as one prompt).  Options by keyword are
        GenerationParams fields (max_tokens, temperature, top_k, top_p, repetition_penalty,
        seed, stop_tokens, ...)."""
        if prompts and isinstance(prompts[0], int):
            prompts = [prompts]
        if params is None:
            params = GenerationParams(**options)
        elif options:
            raise ValueError("give either params or keyword options")
        for i, p in enumerate(prompts):
            if len(p) + params.max_tokens > self.max_context:
                raise ValueError(f"prompt {i} ({len(p)} tokens) plus max_tokens {params.max_tokens} exceeds "
                                 f"max_context {self.max_context}")
        return self._generator.generate(prompts, params, on_token=on_token)

    def benchmark(self, prompts: Sequence[Sequence[int]], max_tokens: int) -> BenchmarkResult:
        """Warm-up prefill, then a timed prefill and a timed greedy decode of exactly
        `max_tokens` tokens per prompt with stop tokens off (TextGenerator.cs:126-186)."""
        if prompts and isinstance(prompts[0], int):
            prompts = [prompts]
        params = GenerationParams.greedy(max_tokens=max_tokens, stop_tokens=())
        warm = GenerationParams.greedy(max_tokens=min(2, max_tokens), stop_tokens=())
        self._generator.generate(prompts, warm)
        torch.cuda.synchronize()
        res = self._generator.generate(prompts, params)
        return BenchmarkResult(res.prompt_tokens, res.generated_tokens, res.prefill_seconds, res.decode_seconds)
