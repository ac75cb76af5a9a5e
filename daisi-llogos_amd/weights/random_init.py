"""Random weights for a configuration and a seed, written as a model folder
(config.json + model.safetensors).  Matrices, tables and biases N(0, 0.02), norm weights
1 + U(-0.1, 0.1).  The reference has no such mode (its tests use real files,
tests/Daisi.Llogos.Tests/TestConstants.cs:16-31)."""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Tuple

import torch

from ..config.registry import architecture_of
from ..models.model import Model
from ..parts.base import TensorSpec
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _generator(seed: int, name: str) -> torch.Generator:
    """A stream per tensor, keyed by seed and name, so a tensor's values do not depend on
    which other tensors the model has."""
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return g


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, std: float = 0.02) -> torch.Tensor:
    g = _generator(seed, spec.name)
    if spec.kind == "norm":
        t = 1.0 + (torch.rand(spec.shape, generator=g, dtype=torch.float32) * 0.2 - 0.1)
    else:
        t = torch.randn(spec.shape, generator=g, dtype=torch.float32) * std
    return t.to(dtype)


def random_tensors(model: Model, seed: int, dtype: torch.dtype, std: float = 0.02) -> Iterator[Tuple[str, torch.Tensor]]:
    for spec in model.tensor_specs():
        yield spec.name, random_tensor(spec, seed, dtype, std)


def write_random_model(folder: str, config: dict, seed: int = 0, std: float = 0.02) -> str:
    """Make `folder` a model folder for the parsed config.json `config`, with random weights
    stored in the configuration's `torch_dtype`.  Returns the folder."""
    arch = architecture_of(config)
    typed = arch.read_config(config)
    model = Model(arch.model_spec(typed))
    store = _STORE.get(str(config.get("torch_dtype", "bfloat16")))
    if store is None:
        raise ValueError(f"torch_dtype {config.get('torch_dtype')!r} cannot be stored (bfloat16, float32, float16)")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh, indent=2)
    layout = [(s.name, tuple(s.shape), store) for s in model.tensor_specs()]
    write_safetensors(os.path.join(folder, "model.safetensors"), random_tensors(model, seed, store, std), layout)
    return folder
