"""Random weights for a configuration and a seed, written as a model folder
(config.json + model.safetensors), or made on the GPU without a folder (the same values).
Matrices, tables and biases N(0, 0.02), norm weights 1 + U(-0.1, 0.1).  The reference has no such mode (its tests use real files,
tests/Daisi.Llogos.Tests/TestConstants.cs:16-31)."""
from __future__ import annotations

import hashlib
import json
import math
import os
from typing import Dict, Iterator, Tuple, Union

import torch

from ..config.registry import architecture_of
from ..models.model import Model
from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


_MASK32 = 0xFFFFFFFF
_CHUNK = {"cpu": 1 << 20, "cuda": 1 << 26}     # elements made at a time (on the CPU what stays in the caches)


def _keys(seed: int, name: str) -> Tuple[int, int]:
    """Two 32-bit keys per tensor, from seed and name, so a tensor's values do not depend on
    which other tensors the model has."""
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:4], "little"), int.from_bytes(digest[4:8], "little")


def _mix32(x: torch.Tensor) -> torch.Tensor:
    """A 32-bit integer hash on int64 tensors (values stay below 2^32; products wrap in 64 bits,
    whose low 32 bits are exact).  Integer arithmetic only: the same bits on any device."""
    x = (x ^ (x >> 16)) * 0x7FEB352D & _MASK32
    x = (x ^ (x >> 15)) * 0x846CA68B & _MASK32
    return x ^ (x >> 16)


def _random_chunk(first: int, count: int, keys: Tuple[int, int], kind: str, std: float, device) -> torch.Tensor:
    """Values of elements first .. first + count - 1 of a tensor, float64: a counter-based
    stream, element i's value depends on (keys, i) alone.  'norm': 1 + U(-0.1, 0.1); anything
    else N(0, std) by Box-Muller from two 24-bit uniforms."""
    idx = torch.arange(first, first + count, dtype=torch.int64, device=device)
    a = _mix32(_mix32((idx + keys[0]) & _MASK32) ^ keys[1])
    u1 = (a >> 8).to(torch.float64)
    if kind == "norm":
        return 1.0 + (u1 * (0.2 / (1 << 24)) - 0.1)
    b = _mix32(a ^ 0x9E3779B9)
    u2 = (b >> 8).to(torch.float64) * (1.0 / (1 << 24))
    radius = torch.sqrt(-2.0 * torch.log((u1 + 1.0) * (1.0 / (1 << 24))))          # u in (0, 1]
    return radius * torch.cos((2.0 * math.pi) * u2) * std


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, std: float = 0.02,
                  device: Union[str, torch.device] = "cpu") -> torch.Tensor:
    """The tensor `spec` of the model with seed `seed`, made on `device`.  The integers behind
    every value are the same on every device; the float64 logarithm and cosine may differ in
    their last bit between devices, which survives the rounding to `dtype` about once in 2^44
    elements for bfloat16: a model made on the GPU is the model written to a folder."""
    keys = _keys(seed, spec.name)
    n = 1
    for d in spec.shape:
        n *= int(d)
    out = torch.empty(n, dtype=dtype, device=device)
    chunk = _CHUNK.get(torch.device(device).type, 1 << 20)
    for first in range(0, n, chunk):
        count = min(chunk, n - first)
        out[first:first + count] = _random_chunk(first, count, keys, spec.kind, std, device).to(dtype)
    return out.view(tuple(spec.shape))


def random_tensors(model: Model, seed: int, dtype: torch.dtype, std: float = 0.02,
                   device: Union[str, torch.device] = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for spec in model.tensor_specs():
        yield spec.name, random_tensor(spec, seed, dtype, std, device)


def storage_dtype(config: dict) -> torch.dtype:
    store = _STORE.get(str(config.get("torch_dtype", "bfloat16")))
    if store is None:
        raise ValueError(f"torch_dtype {config.get('torch_dtype')!r} cannot be stored (bfloat16, float32, float16)")
    return store


def write_random_model(folder: str, config: dict, seed: int = 0, std: float = 0.02,
                       device: Union[str, torch.device] = "cpu") -> str:
    """Make `folder` a model folder for the parsed config.json `config`, with random weights
    stored in the configuration's `torch_dtype`.  Returns the folder.  `device` is where the
    numbers are made (a GPU makes a large model in seconds; the values are the same)."""
    arch = architecture_of(config)
    typed = arch.read_config(config)
    model = Model(arch.model_spec(typed))
    store = storage_dtype(config)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh, indent=2)
    layout = [(s.name, tuple(s.shape), store) for s in model.tensor_specs()]
    write_safetensors(os.path.join(folder, "model.safetensors"), random_tensors(model, seed, store, std, device), layout)
    return folder
