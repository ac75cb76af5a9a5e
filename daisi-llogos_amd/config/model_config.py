"""Typed configuration of the dense decoder, read from config.json.

The reference reads the same quantities from GGUF metadata
(src/dotnet/Daisi.Llogos/Model/ModelConfig.cs:124-201: block_count, embedding_length,
feed_forward_length, context_length, layer_norm_rms_epsilon default 1e-6, head_count,
head_count_kv, key_length default hidden/heads, rope.freq_base default 10000,
rope.dimension_count) and raises on a missing key (:218-250).  Here the keys are the
ones a config.json of this architecture carries.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field
from typing import Any, Optional


class ConfigError(ValueError):
    """A config.json that cannot describe a model: missing key, wrong type, impossible sizes."""


_MISSING = object()


class ConfigReader:
    """Typed getters over a parsed config.json; every error names the key."""

    def __init__(self, data: dict, source: str = "config.json"):
        if not isinstance(data, dict):
            raise ConfigError(f"{source}: top level must be an object")
        self.data = data
        self.source = source

    def _raw(self, key: str, default: Any = _MISSING) -> Any:
        if key not in self.data or self.data[key] is None:
            if default is _MISSING:
                raise ConfigError(f"{self.source}: missing key '{key}'")
            return default
        return self.data[key]

    def int(self, key: str, default: Any = _MISSING) -> int:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
            raise ConfigError(f"{self.source}: key '{key}' must be an integer, got {v!r}")
        return int(v)

    def float(self, key: str, default: Any = _MISSING) -> float:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.source}: key '{key}' must be a number, got {v!r}")
        return float(v)

    def bool(self, key: str, default: Any = _MISSING) -> bool:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, bool):
            raise ConfigError(f"{self.source}: key '{key}' must be true or false, got {v!r}")
        return v

    def str(self, key: str, default: Any = _MISSING) -> str:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, str):
            raise ConfigError(f"{self.source}: key '{key}' must be a string, got {v!r}")
        return v

    def int_list(self, key: str, default: Any = _MISSING) -> list:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        items = v if isinstance(v, list) else [v]
        out = []
        for it in items:
            if isinstance(it, bool) or not isinstance(it, int):
                raise ConfigError(f"{self.source}: key '{key}' must hold integers, got {v!r}")
            out.append(int(it))
        return out

    def obj(self, key: str, default: Any = _MISSING) -> Optional[dict]:
        v = self._raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, dict):
            raise ConfigError(f"{self.source}: key '{key}' must be an object, got {v!r}")
        return v


@dataclass(frozen=True)
class RopeScaling:
    """Frequency scaling rule of the rotary encoding (config key `rope_scaling`)."""
    rope_type: str
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    def to_json(self) -> dict:
        d = {"rope_type": self.rope_type, "factor": self.factor}
        if self.rope_type == "llama3":
            d.update(low_freq_factor=self.low_freq_factor, high_freq_factor=self.high_freq_factor,
                     original_max_position_embeddings=self.original_max_position_embeddings)
        return d


@dataclass(frozen=True)
class DenseDecoderConfig:
    """Every size and constant of a Llama / Qwen2 / Qwen3 dense decoder."""
    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    partial_rotary_factor: float = 1.0
    rope_scaling: Optional[RopeScaling] = None
    max_position_embeddings: int = 2048
    attention_bias: bool = False
    qk_norm: bool = False
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: int = 0
    max_window_layers: int = 0
    torch_dtype: str = "bfloat16"
    bos_token_id: Optional[int] = None
    eos_token_ids: tuple = field(default_factory=tuple)

    # ---- derived quantities -------------------------------------------------
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def rotary_dim(self) -> int:
        return int(self.head_dim * self.partial_rotary_factor)

    def layer_window(self, layer: int) -> int:
        """Window of a layer's attention, 0 for all keys.  Layers from `max_window_layers`
        on are windowed when `use_sliding_window` is set."""
        if self.use_sliding_window and self.sliding_window > 0 and layer >= self.max_window_layers:
            return self.sliding_window
        return 0

    def validate(self) -> None:
        pos = ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
               "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"]
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError(f"config: '{k}' must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config: num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        from ..cache.pages import HEAD_DIM_STEP, MAX_HEAD_DIM
        if self.head_dim % HEAD_DIM_STEP or self.head_dim > MAX_HEAD_DIM:
            how = "given as 'head_dim'" if self.head_dim * self.num_attention_heads != self.hidden_size else \
                f"hidden_size {self.hidden_size} / num_attention_heads {self.num_attention_heads}"
            raise ConfigError(f"config: 'head_dim' ({self.head_dim}, {how}) must be a multiple of {HEAD_DIM_STEP}, "
                              f"at most {MAX_HEAD_DIM}: the cache's pages and the attention kernels work in "
                              f"fragments of {HEAD_DIM_STEP} dimensions")
        if self.rotary_dim <= 0 or self.rotary_dim % 2 != 0 or self.rotary_dim > self.head_dim:
            raise ConfigError(f"config: rotary dimension {self.rotary_dim} must be even and within head_dim")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"config: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"config: rope_theta must be positive, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(f"config: hidden_act '{self.hidden_act}' is not supported (silu only)")
        if self.rope_scaling is not None and self.rope_scaling.rope_type not in ("llama3", "linear", "default"):
            raise ConfigError(f"config: rope_scaling type '{self.rope_scaling.rope_type}' is not supported")
        if self.use_sliding_window and self.sliding_window <= 0:
            raise ConfigError("config: use_sliding_window needs a positive sliding_window")

    # ---- reading and writing -------------------------------------------------
    @classmethod
    def from_dict(cls, data: dict, *, attention_bias_default: bool = False, qk_norm: bool = False,
                  source: str = "config.json") -> "DenseDecoderConfig":
        r = ConfigReader(data, source)
        archs = r._raw("architectures")
        if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
            raise ConfigError(f"{source}: key 'architectures' must be a list of names")
        hidden = r.int("hidden_size")
        heads = r.int("num_attention_heads")
        if heads <= 0:
            raise ConfigError(f"{source}: num_attention_heads must be positive")
        head_dim = r.int("head_dim", None)
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(f"{source}: hidden_size {hidden} is not a multiple of num_attention_heads "
                                  f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        scaling = None
        rs = r.obj("rope_scaling", None)
        if rs is not None:
            rr = ConfigReader(rs, source + ":rope_scaling")
            rtype = rr.str("rope_type", None) or rr.str("type")
            scaling = RopeScaling(
                rope_type=rtype,
                factor=rr.float("factor", 1.0),
                low_freq_factor=rr.float("low_freq_factor", 1.0),
                high_freq_factor=rr.float("high_freq_factor", 4.0),
                original_max_position_embeddings=rr.int("original_max_position_embeddings", 8192))
        cfg = cls(
            architecture=archs[0],
            vocab_size=r.int("vocab_size"),
            hidden_size=hidden,
            intermediate_size=r.int("intermediate_size"),
            num_hidden_layers=r.int("num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=r.int("num_key_value_heads", heads),
            head_dim=head_dim,
            rms_norm_eps=r.float("rms_norm_eps", 1e-6),
            rope_theta=r.float("rope_theta", 10000.0),
            partial_rotary_factor=r.float("partial_rotary_factor", 1.0),
            rope_scaling=scaling,
            max_position_embeddings=r.int("max_position_embeddings", 2048),
            attention_bias=r.bool("attention_bias", attention_bias_default),
            qk_norm=qk_norm,
            tie_word_embeddings=r.bool("tie_word_embeddings", False),
            hidden_act=r.str("hidden_act", "silu"),
            use_sliding_window=r.bool("use_sliding_window", False),
            sliding_window=r.int("sliding_window", 0),
            max_window_layers=r.int("max_window_layers", 0),
            torch_dtype=r.str("torch_dtype", None) or r.str("dtype", "bfloat16"),
            bos_token_id=r.int("bos_token_id", None),
            eos_token_ids=tuple(r.int_list("eos_token_id", [])),
        )
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        d = {
            "architectures": [self.architecture],
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "attention_bias": self.attention_bias,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "torch_dtype": self.torch_dtype,
        }
        if self.partial_rotary_factor != 1.0:
            d["partial_rotary_factor"] = self.partial_rotary_factor
        if self.rope_scaling is not None:
            d["rope_scaling"] = self.rope_scaling.to_json()
        if self.use_sliding_window:
            d.update(use_sliding_window=True, sliding_window=self.sliding_window,
                     max_window_layers=self.max_window_layers)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return d

    def replace(self, **kw) -> "DenseDecoderConfig":
        cfg = dataclasses.replace(self, **kw)
        cfg.validate()
        return cfg


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder '{folder}'")
    try:
        with open(path) as fh:
            return json.load(fh)
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from e
