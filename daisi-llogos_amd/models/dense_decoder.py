"""The Llama / Qwen2 / Qwen3 dense decoder as a ModelSpec: which parts make a layer, with
which sizes, and under which tensor names.

Tensor names follow the config.json + safetensors convention; the reference's GGUF names
map onto them one to one (Daisi.Llogos/Model/ModelLoader.cs:17-19, 94-113):
token_embd -> model.embed_tokens, blk.N.attn_norm -> input_layernorm, attn_q/k/v/output ->
self_attn.{q,k,v,o}_proj, attn_q_norm/attn_k_norm -> self_attn.{q,k}_norm,
post_attention_norm | ffn_norm -> post_attention_layernorm, ffn_gate/up/down ->
mlp.{gate,up,down}_proj, output_norm -> model.norm, output -> lm_head (absent: the
embedding serves, Daisi.Llogos/Model/ModelWeights.cs:29).
"""
from __future__ import annotations

from typing import Optional

from ..config.model_config import DenseDecoderConfig
from ..parts.rope import Rotary
from .model import LayerSpec, ModelSpec


def dense_decoder_spec(cfg: DenseDecoderConfig, *, attention_window: Optional[int] = None,
                       attention_sinks: int = 0, rotary_pairing: str = "split_half") -> ModelSpec:
    """`attention_window` / `attention_sinks` override the configuration's windows for every
    layer (the reference's run-time attention strategy,
    Daisi.Llogos/Inference/AttentionStrategy.cs:75-100)."""
    scaling = cfg.rope_scaling.to_json() if cfg.rope_scaling is not None else None
    rotary = Rotary(cfg.head_dim, cfg.rotary_dim, cfg.rope_theta, pairing=rotary_pairing, scaling=scaling)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        window = cfg.layer_window(i) if attention_window is None else attention_window
        layers.append(LayerSpec(
            mixer=("attention", dict(prefix=p + "self_attn.", hidden=cfg.hidden_size,
                                     n_heads=cfg.num_attention_heads, n_kv_heads=cfg.num_key_value_heads,
                                     head_dim=cfg.head_dim, position=rotary, bias=cfg.attention_bias,
                                     qk_norm=cfg.qk_norm, eps=cfg.rms_norm_eps, window=window,
                                     sinks=attention_sinks if window else 0)),
            ffn=("swiglu", dict(prefix=p + "mlp.", hidden=cfg.hidden_size, intermediate=cfg.intermediate_size)),
            mixer_norm=("rmsnorm", dict(name=p + "input_layernorm", width=cfg.hidden_size, eps=cfg.rms_norm_eps)),
            ffn_norm=("rmsnorm", dict(name=p + "post_attention_layernorm", width=cfg.hidden_size,
                                      eps=cfg.rms_norm_eps)),
        ))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="model.embed_tokens.weight",
        layers=layers,
        final_norm=("rmsnorm", dict(name="model.norm", width=cfg.hidden_size, eps=cfg.rms_norm_eps)),
        head_name="lm_head", tie_head=cfg.tie_word_embeddings,
        eos_token_ids=tuple(cfg.eos_token_ids), max_position=cfg.max_position_embeddings)
