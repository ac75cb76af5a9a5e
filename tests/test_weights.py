"""Weights by name: reading, the one error that lists every difference, random mode."""
import json
import os

import pytest
import torch

import tiny_configs as tc


def _folder(llogos, tmp_path, cfg=tc.TINY_A, seed=0):
    return llogos.write_random_model(str(tmp_path / "model"), cfg, seed=seed)


def _rewrite(folder, change):
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    change(tensors)
    save_file(tensors, path)


def _model(llogos, cfg):
    arch = llogos.architecture_of(cfg)
    return llogos.Model(arch.model_spec(arch.read_config(cfg)))


def test_random_folder_reads_back_like_the_library(llogos, tmp_path):
    from safetensors.torch import load_file
    folder = _folder(llogos, tmp_path)
    ref = load_file(os.path.join(folder, "model.safetensors"))
    ck = llogos.Checkpoint(folder)
    assert set(ck.shapes()) == set(ref)
    for name, t in ref.items():
        got = ck.get(name)
        assert got.dtype == torch.bfloat16 and torch.equal(got, t)
    assert ck.get("nope") is None
    ck.check(_model(llogos, tc.TINY_A).tensor_specs())
    ck.close()


def test_random_mode_is_reproducible_and_seeded(llogos, tmp_path):
    a = llogos.Checkpoint(_folder(llogos, tmp_path / "a", seed=5))
    b = llogos.Checkpoint(_folder(llogos, tmp_path / "b", seed=5))
    c = llogos.Checkpoint(_folder(llogos, tmp_path / "c", seed=6))
    n = "model.layers.1.mlp.down_proj.weight"
    assert torch.equal(a.get(n), b.get(n)) and not torch.equal(a.get(n), c.get(n))
    w = a.get(n).float()
    assert abs(w.std().item() - 0.02) < 0.003 and abs(w.mean().item()) < 0.003
    g = a.get("model.norm.weight").float()
    assert 0.9 <= g.min().item() and g.max().item() <= 1.1 and g.std().item() > 0.01
    assert a.get("model.layers.0.self_attn.k_proj.bias").float().abs().max().item() > 0
    assert json.load(open(os.path.join(a.folder, "config.json"))) == tc.TINY_A


def test_storage_types(llogos, tmp_path):
    f32 = llogos.Checkpoint(_folder(llogos, tmp_path / "f", dict(tc.TINY_A, torch_dtype="float32")))
    assert f32.get("model.norm.weight").dtype == torch.float32          # a tensor stored in 32-bit stays so
    folder = _folder(llogos, tmp_path / "i")
    _rewrite(folder, lambda t: t.update(position_ids=torch.arange(7, dtype=torch.int64)))
    ck = llogos.Checkpoint(folder)
    assert ck.get("position_ids").dtype == torch.int32                   # integer tables as int32
    assert ck.get("model.norm.weight").dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(llogos, tmp_path):
    folder = _folder(llogos, tmp_path)

    def change(t):
        del t["model.layers.0.mlp.up_proj.weight"]
        del t["model.layers.1.self_attn.q_proj.bias"]
        t["model.layers.0.self_attn.rotary.extra"] = torch.zeros(3)
        t["model.layers.1.mlp.down_proj.weight"] = torch.zeros(64, 175, dtype=torch.bfloat16)
        t["model.norm.weight"] = torch.zeros(63, dtype=torch.bfloat16)
    _rewrite(folder, change)
    ck = llogos.Checkpoint(folder)
    with pytest.raises(llogos.WeightError) as ei:
        ck.check(_model(llogos, tc.TINY_A).tensor_specs())
    e = ei.value
    assert e.missing == ["model.layers.0.mlp.up_proj.weight", "model.layers.1.self_attn.q_proj.bias"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary.extra"]
    assert len(e.wrong_shape) == 2 and "expected [64, 176], found [64, 175]" in str(e)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "model.norm.weight"):
        assert word in str(e)


def test_options_are_checked_against_the_checkpoint(llogos, tmp_path):
    # a Qwen3 checkpoint read as Llama: the q/k norms are unexpected; as Qwen2: biases are missing
    folder = _folder(llogos, tmp_path, tc.TINY_B)
    ck = llogos.Checkpoint(folder)
    with pytest.raises(llogos.WeightError, match="q_norm"):
        ck.check(_model(llogos, dict(tc.TINY_B, architectures=["LlamaForCausalLM"])).tensor_specs())
    with pytest.raises(llogos.WeightError, match="q_proj.bias"):
        ck.check(_model(llogos, dict(tc.TINY_B, architectures=["Qwen2ForCausalLM"])).tensor_specs())
    # an untied configuration needs its head
    with pytest.raises(llogos.WeightError, match="lm_head.weight"):
        ck.check(_model(llogos, dict(tc.TINY_B, tie_word_embeddings=False)).tensor_specs())


def test_tied_checkpoint_may_store_its_head(llogos, tmp_path):
    folder = _folder(llogos, tmp_path, tc.TINY_B)
    _rewrite(folder, lambda t: t.update({"lm_head.weight": t["model.embed_tokens.weight"].clone()}))
    ck = llogos.Checkpoint(folder)
    ck.check(_model(llogos, tc.TINY_B).tensor_specs(), tied_head="lm_head.weight")
    with pytest.raises(llogos.WeightError, match="unexpected"):
        ck.check(_model(llogos, tc.TINY_B).tensor_specs())


def test_broken_files(llogos, tmp_path):
    io = __import__("importlib").import_module("daisi-llogos_amd.weights.safetensors_io")
    with pytest.raises(io.SafetensorsError, match="model.safetensors"):
        llogos.Checkpoint(str(tmp_path))
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x00\x01")
    with pytest.raises(io.SafetensorsError, match="short"):
        llogos.Checkpoint(str(tmp_path))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(io.SafetensorsError, match="header"):
        llogos.Checkpoint(str(tmp_path))


def test_sharded_checkpoint(llogos, tmp_path):
    from safetensors.torch import load_file, save_file
    folder = _folder(llogos, tmp_path)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    names = sorted(tensors)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for fname, ns in shards.items():
        save_file({n: tensors[n] for n in ns}, os.path.join(folder, fname))
    os.remove(path)
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as fh:
        json.dump({"weight_map": {n: f for f, ns in shards.items() for n in ns}}, fh)
    ck = llogos.Checkpoint(folder)
    ck.check(_model(llogos, tc.TINY_A).tensor_specs())
    assert torch.equal(ck.get(names[-1]), tensors[names[-1]])
