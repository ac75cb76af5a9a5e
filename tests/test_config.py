"""Configuration and registry: keys, defaults, errors."""
import copy
import json

import pytest

import tiny_configs as tc


def test_every_size_comes_from_config_json(llogos):
    arch = llogos.architecture_of(tc.TINY_B)
    cfg = arch.read_config(tc.TINY_B)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size) == (3, 96, 288)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (6, 1, 32)
    assert cfg.q_width == 192 and cfg.kv_width == 32 and cfg.rotary_dim == 32
    assert cfg.vocab_size == 384 and cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6
    assert cfg.tie_word_embeddings and cfg.qk_norm and not cfg.attention_bias
    assert cfg.eos_token_ids == (382, 383) and cfg.max_position_embeddings == 256


def test_defaults_of_the_reference(llogos):
    # eps 1e-6, theta 10000, kv heads = heads, head_dim = hidden / heads
    # (Daisi.Llogos/Model/ModelConfig.cs:170-181)
    d = {"architectures": ["LlamaForCausalLM"], "vocab_size": 10, "hidden_size": 32, "intermediate_size": 48,
         "num_hidden_layers": 1, "num_attention_heads": 2}
    cfg = llogos.architecture_of(d).read_config(d)
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 10000.0
    assert cfg.num_key_value_heads == 2 and cfg.head_dim == 16 and cfg.rope_scaling is None
    assert not cfg.attention_bias and not cfg.qk_norm and not cfg.tie_word_embeddings


def test_architecture_defaults_and_override(llogos):
    a = llogos.architecture_of(tc.TINY_A).read_config(tc.TINY_A)
    assert a.attention_bias and not a.qk_norm
    d = dict(tc.TINY_A, attention_bias=False)
    assert not llogos.architecture_of(d).read_config(d).attention_bias
    d = dict(tc.TINY_C, attention_bias=True)
    assert llogos.architecture_of(d).read_config(d).attention_bias
    assert set(llogos.ARCHITECTURES) >= {"LlamaForCausalLM", "Qwen2ForCausalLM", "Qwen3ForCausalLM"}


def test_rope_scaling_and_window_keys(llogos):
    c = llogos.architecture_of(tc.TINY_C).read_config(tc.TINY_C)
    assert c.rope_scaling.rope_type == "llama3" and c.rope_scaling.factor == 8.0
    assert c.rope_scaling.original_max_position_embeddings == 64
    w = llogos.architecture_of(tc.TINY_W).read_config(tc.TINY_W)
    assert [w.layer_window(i) for i in range(3)] == [0, 70, 70]
    d = dict(tc.TINY_W, use_sliding_window=False)
    assert llogos.architecture_of(d).read_config(d).layer_window(2) == 0


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads"])
def test_missing_key_is_named(llogos, key):
    d = copy.deepcopy(tc.TINY_A)
    del d[key]
    with pytest.raises(llogos.ConfigError, match=key):
        llogos.architecture_of(d).read_config(d)


def test_wrong_types_and_sizes(llogos):
    def read(**kw):
        d = dict(tc.TINY_A, **kw)
        return llogos.architecture_of(d).read_config(d)
    with pytest.raises(llogos.ConfigError, match="hidden_size"):
        read(hidden_size="64")
    with pytest.raises(llogos.ConfigError, match="integer"):
        read(num_hidden_layers=2.5)
    assert read(num_hidden_layers=2.0).num_hidden_layers == 2           # whole floats are accepted
    with pytest.raises(llogos.ConfigError, match="multiple"):
        read(num_key_value_heads=3)
    with pytest.raises(llogos.ConfigError, match="head_dim"):
        read(hidden_size=66)                                            # 66 / 4 heads and no head_dim
    # head sizes are refused where the configuration is read, with the key's name: a multiple of 16 ...
    with pytest.raises(llogos.ConfigError, match=r"'head_dim' \(40, hidden_size 320 / num_attention_heads 8\) must be a multiple of 16"):
        read(hidden_size=320, num_attention_heads=8, num_key_value_heads=8)
    with pytest.raises(llogos.ConfigError, match=r"'head_dim' \(24, given as 'head_dim'\)"):
        read(head_dim=24)
    with pytest.raises(llogos.ConfigError, match="at most 512"):
        read(head_dim=528)                                              # ... within what the attention kernels take
    assert read(head_dim=48).head_dim == 48
    with pytest.raises(llogos.ConfigError, match="rms_norm_eps"):
        read(rms_norm_eps=0)
    with pytest.raises(llogos.ConfigError, match="hidden_act"):
        read(hidden_act="gelu")
    with pytest.raises(llogos.ConfigError, match="rope_scaling"):
        read(rope_scaling={"rope_type": "yarn", "factor": 2.0})
    with pytest.raises(llogos.ConfigError, match="tie_word_embeddings"):
        read(tie_word_embeddings="yes")


def test_unknown_architecture_lists_known(llogos):
    with pytest.raises(llogos.ConfigError, match="LlamaForCausalLM"):
        llogos.architecture_of({"architectures": ["MambaForCausalLM"]})
    with pytest.raises(llogos.ConfigError, match="architectures"):
        llogos.architecture_of({"hidden_size": 3})


def test_missing_config_file(llogos, tmp_path):
    with pytest.raises(llogos.ConfigError, match="config.json"):
        llogos.read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(llogos.ConfigError, match="JSON"):
        llogos.read_config_json(str(tmp_path))


def test_round_trip(llogos):
    for d in tc.ALL.values():
        cfg = llogos.architecture_of(d).read_config(d)
        again = llogos.architecture_of(cfg.to_dict()).read_config(json.loads(json.dumps(cfg.to_dict())))
        assert again == cfg


def test_model_spec_follows_the_configuration(llogos):
    cfg = llogos.architecture_of(tc.TINY_W).read_config(tc.TINY_W)
    model = llogos.Model(llogos.dense_decoder_spec(cfg))
    assert [l.mixer.window for l in model.layers] == [0, 70, 70]
    needs = model.cache_needs()
    assert len({kv for kv, _ in needs}) == 2 and all(st is None for _, st in needs)
    names = {s.name for s in model.tensor_specs()}
    assert "model.layers.2.self_attn.q_proj.bias" in names and "lm_head.weight" in names
    b = llogos.architecture_of(tc.TINY_B).read_config(tc.TINY_B)
    nb = {s.name: s.shape for s in llogos.Model(llogos.dense_decoder_spec(b)).tensor_specs()}
    assert "lm_head.weight" not in nb and nb["model.layers.0.self_attn.q_norm.weight"] == (32,)
    assert nb["model.layers.1.self_attn.q_proj.weight"] == (192, 96)
    assert nb["model.layers.1.self_attn.o_proj.weight"] == (96, 192)
