"""daisi-llogos_amd: a small MI355X-native inference library for the Llama / Qwen2 / Qwen3
dense decoder: configuration, weights, parts, cache, step function, generation, sampling,
hand-written HIP kernels for gfx950.

The directory name is no Python identifier; import the package with
    importlib.import_module("daisi-llogos_amd")
"""
from . import parts as parts                      # registers the built-in parts
from .config import (ARCHITECTURES, ConfigError, DenseDecoderConfig, RopeScaling, architecture_of,
                     read_config_json, register_architecture)
from .weights import Checkpoint, WeightError, write_random_model
from .models import LayerSpec, Model, ModelSpec, ScheduleEntry, dense_decoder_spec
from .cache import Cache, CacheError, CacheFull
from .engine import Engine, GenerationResult, Generator, StepError, StepProbe, plan_batches
from .sampling import GenerationParams, Sampler
from .api import BenchmarkResult, Llogos, parse_attention

__all__ = [
    "ARCHITECTURES", "ConfigError", "DenseDecoderConfig", "RopeScaling", "architecture_of", "read_config_json",
    "register_architecture", "Checkpoint", "WeightError", "write_random_model", "LayerSpec", "Model",
    "ModelSpec", "ScheduleEntry", "dense_decoder_spec", "Cache", "CacheError", "CacheFull", "Engine", "StepError", "StepProbe",
    "GenerationResult", "Generator", "plan_batches", "GenerationParams", "Sampler", "BenchmarkResult", "Llogos",
    "parse_attention",
]
