"""One registry from an architecture's name (config.json `architectures[0]`) to the
functions that read its configuration and describe its model.

The reference switches on the GGUF `general.architecture` string; llama, qwen2 and qwen3
all take its standard path and their optional features are found by tensor presence
(Daisi.Llogos.Cli/Program.cs:54-57, 101-103; Daisi.Llogos/Model/ModelLoader.cs:106-110).
Here each name states its defaults, and the loader checks them against the checkpoint."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from .model_config import ConfigError, DenseDecoderConfig


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[dict], object]        # parsed config.json -> typed configuration
    model_spec: Callable[..., object]            # typed configuration (+ options) -> ModelSpec


ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, read_config: Callable[[dict], object],
                          model_spec: Callable[..., object]) -> Architecture:
    arch = Architecture(name, read_config, model_spec)
    ARCHITECTURES[name] = arch
    return arch


def architecture_of(data: dict) -> Architecture:
    archs = data.get("architectures") if isinstance(data, dict) else None
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json: missing key 'architectures' (a list with the model's class name)")
    name = archs[0]
    if name not in ARCHITECTURES:
        raise ConfigError(f"unknown architecture '{name}'; known: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[name]


def _dense(name: str, bias_default: bool, qk_norm: bool) -> None:
    from ..models.dense_decoder import dense_decoder_spec

    def read(data: dict) -> DenseDecoderConfig:
        return DenseDecoderConfig.from_dict(data, attention_bias_default=bias_default, qk_norm=qk_norm)
    register_architecture(name, read, dense_decoder_spec)


_dense("LlamaForCausalLM", bias_default=False, qk_norm=False)
_dense("Qwen2ForCausalLM", bias_default=True, qk_norm=False)
_dense("Qwen3ForCausalLM", bias_default=False, qk_norm=True)
