"""The Python entry point: load a model folder, generate, benchmark.

The reference's entry points are TextGenerator.Generate / Benchmark
(Daisi.Llogos/Inference/TextGenerator.cs:26-186) behind its command line
(Daisi.Llogos.Cli/Program.cs); option names and defaults follow them."""
from __future__ import annotations

import re
import time
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple, Union

import torch

from .cache.pages import PAGE_TOKENS, pages_for
from .engine.generate import GenerationResult, Generator
from .engine.step import Engine
from .sampling.params import GenerationParams


_ATTENTION_FORMS = re.compile(r"^(?:(full)|window:(\d+)|sinks:(\d+),(\d+))$")


# Published peaks by GPU architecture name: memory bytes a second, dense matrix flops a second by type.
# A GPU that is not listed here has no peaks, and fractions of peak are reported as 0 for it.
DEVICE_PEAKS = {
    "gfx950": {"hbm": 8.0e12, "bf16": 2.5e15, "fp32": 157.3e12},           # MI355X
}


def device_peaks(device: Union[str, torch.device, int, None] = None) -> dict:
    """The published peaks of the GPU `device` (the current one when None), {} when unknown."""
    if not torch.cuda.is_available():
        return {}
    name = torch.cuda.get_device_properties(torch.device(device) if device is not None else torch.cuda.current_device())
    arch = getattr(name, "gcnArchName", "").split(":")[0]
    return DEVICE_PEAKS.get(arch, {})


def parse_attention(value: str) -> Tuple[Optional[int], int]:
    """The command line's --attention option: 'full' (the configuration's own attention),
    'window:N' (the last N positions) or 'sinks:S,W' (the first S positions and the last W), the
    reference's three strategies (Daisi.Llogos/Inference/AttentionStrategy.cs:75-100).
    Returns (positions the cache keeps for a sequence, or None for 'full'; how many of them are sinks)."""
    m = _ATTENTION_FORMS.match(value.strip().lower())
    if m is None:
        raise ValueError(f"--attention takes full, window:<N> or sinks:<S>,<W>, not '{value}'")
    if m.group(1):
        return None, 0
    sinks, window = (0, int(m.group(2))) if m.group(2) is not None else (int(m.group(3)), int(m.group(4)))
    if window == 0:
        raise ValueError(f"--attention {value}: the window must hold at least one position")
    return sinks + window, sinks


@dataclass
class BenchmarkResult:
    """As the reference's BenchmarkResult (TextGenerator.cs:238-247), summed over the batch."""
    prompt_tokens: int
    generated_tokens: int
    prefill_seconds: float
    decode_seconds: float
    prefill_flops: float = 0.0            # of the timed prompt step
    decode_bytes: float = 0.0             # every decode step's weights once + the cache of its live sequences
    dtype: str = "bf16"
    peaks: Optional[dict] = None          # device_peaks() of the GPU it ran on; None: looked up when asked for

    def _peak(self, key: str) -> float:
        peaks = self.peaks if self.peaks is not None else device_peaks()
        return float(peaks.get(key, 0.0))

    @property
    def prefill_tokens_per_second(self) -> float:
        return self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0

    @property
    def decode_tokens_per_second(self) -> float:
        return self.generated_tokens / self.decode_seconds if self.decode_seconds > 0 else 0.0

    @property
    def prefill_fraction_of_peak(self) -> float:
        """Flops of the prompt step / its time / the GPU's published dense matrix peak for the type (0 for
        a GPU whose peaks are not known)."""
        peak = self._peak(self.dtype)
        return self.prefill_flops / self.prefill_seconds / peak if self.prefill_seconds > 0 and peak else 0.0

    @property
    def decode_bytes_per_second(self) -> float:
        return self.decode_bytes / self.decode_seconds if self.decode_seconds > 0 else 0.0

    @property
    def decode_fraction_of_peak(self) -> float:
        """Bytes the decode steps had to read / their time / the GPU's published memory bandwidth (0 for a
        GPU whose peaks are not known)."""
        peak = self._peak("hbm")
        return self.decode_bytes_per_second / peak if peak else 0.0


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
        self.max_batch = max_batch
        self.engine = Engine.from_folder(model, dtype=dtype, max_tokens=pool, n_slots=max(max_batch, 1),
                                         device=device, max_seq=max_context, **options)
        # the engine keeps the limit within the positions the model was made for
        self.max_context = self.engine.max_seq or max_context
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
            # the last generated token is not fed back: a request comes to hold len(p) + max_tokens - 1 positions
            if len(p) + max(params.max_tokens, 1) - 1 > self.max_context:
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
        model, lens = self.engine.model, [len(p) for p in prompts]
        weights, per_position = model.step_weight_bytes(), self.engine.cache.bytes_per_position()
        # decode step t (the prompt step made token 0) reads the weights and, of each sequence, len + t positions
        steps_by_batch = {}
        for batch in res.batches:
            steps_by_batch[len(batch)] = steps_by_batch.get(len(batch), 0) + max(0, max_tokens - 1)
        decode_bytes = sum(n * weights for n in steps_by_batch.values()) + \
            per_position * sum(n + t for n in lens for t in range(1, max_tokens))
        flops = sum(model.step_flops([lens[r] for r in batch], wanted_rows=len(batch)) for batch in res.batches)
        return BenchmarkResult(res.prompt_tokens, res.generated_tokens, res.prefill_seconds, res.decode_seconds,
                               prefill_flops=flops, decode_bytes=decode_bytes,
                               dtype="fp32" if self.engine.rt.is_f32 else "bf16", peaks=device_peaks(self.engine.rt.device))
