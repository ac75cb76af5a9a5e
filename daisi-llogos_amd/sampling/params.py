"""Options of a generation, with the reference's names, meanings and defaults
(Daisi.Llogos/Inference/GenerationParams.cs:6-60)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class GenerationParams:
    max_tokens: int = 256                 # MaxTokens: most new tokens
    temperature: float = 0.8              # Temperature: 0 = greedy (first maximum)
    top_k: int = 40                       # TopK: 0 = off
    top_p: float = 0.95                   # TopP: 1.0 = off
    repetition_penalty: float = 1.1       # RepetitionPenalty: 1.0 = off
    stop_tokens: Optional[Tuple[int, ...]] = None   # StopTokens: None = the model's end-of-sequence ids
    seed: Optional[int] = None            # Seed: None = not reproducible
    frequency_penalty: float = 0.0        # FrequencyPenalty
    presence_penalty: float = 0.0         # PresencePenalty
    min_p: float = 0.0                    # MinP: 0 = off
    typical_p: float = 1.0                # TypicalP: 1.0 = off
    penalize_newline: bool = False        # PenalizeNewline
    penalty_count: int = 64               # PenaltyCount: last tokens the penalties look at, 0 = all
    min_keep: int = 1                     # MinKeep
    prevent_eos: bool = False             # PreventEOS: stop tokens can not be drawn

    def __post_init__(self):
        if self.max_tokens < 0:
            raise ValueError("max_tokens must not be negative")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.top_k < 0:
            raise ValueError("top_k must not be negative")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    @property
    def has_penalties(self) -> bool:
        return self.repetition_penalty != 1.0 or self.frequency_penalty != 0 or self.presence_penalty != 0

    @property
    def is_greedy(self) -> bool:
        """The reference's short cut: temperature 0 and no penalties (Sampler.cs:32-34)."""
        return self.temperature == 0 and not self.has_penalties

    @classmethod
    def greedy(cls, max_tokens: int = 256, **kw) -> "GenerationParams":
        return cls(max_tokens=max_tokens, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, **kw)
