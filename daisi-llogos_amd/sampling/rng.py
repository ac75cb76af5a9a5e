"""Uniform numbers for sampling that depend on (seed, request, token index) alone, so a
request draws the same numbers whatever else is in its batch.  The reference draws from one
System.Random per sampler (Daisi.Llogos/Inference/Sampler.cs:12-15, 336); with one sequence
per sampler that is the same property."""
from __future__ import annotations

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform(seed: int, request: int, index: int) -> float:
    """A float32-exact number in [0, 1): 24 random bits."""
    h = _splitmix64(seed & _MASK)
    h = _splitmix64(h ^ ((request + 1) * 0xD6E8FEB86659FD93 & _MASK))
    h = _splitmix64(h ^ ((index + 1) * 0xA0761D6478BD642F & _MASK))
    return (h >> 40) / float(1 << 24)
