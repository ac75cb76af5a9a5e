"""The command line's options carry the reference's names and defaults
(Daisi.Llogos.Cli/Program.cs:444-530, 800-827)."""
import importlib

import pytest

cli = importlib.import_module("daisi-llogos_amd.__main__")
api = importlib.import_module("daisi-llogos_amd.api")


def test_defaults():
    a = cli.parse_args(["--model", "m", "--prompt", "1 2"])
    assert (a.max_tokens, a.max_context, a.temperature, a.top_k, a.top_p, a.repeat_penalty) == \
           (256, 2048, 0.7, 40, 0.9, 1.1)
    assert a.seed is None and not a.bench and a.attention == "full"


def test_short_and_long_names():
    a = cli.parse_args(["-m", "dir", "-p", "5,6", "-n", "7", "-t", "0", "--top-k", "3", "--top-p", "0.5",
                        "--repeat-penalty", "1.0", "--seed", "9", "--max-context", "128", "--bench", "-b", "hip"])
    assert (a.model, a.prompt, a.max_tokens, a.temperature, a.top_k, a.top_p) == ("dir", "5,6", 7, 0.0, 3, 0.5)
    assert (a.repeat_penalty, a.seed, a.max_context, a.bench, a.backend) == (1.0, 9, 128, True, "hip")
    with pytest.raises(ValueError, match="Missing value"):
        cli.parse_args(["--model"])
    with pytest.raises(ValueError, match="unknown"):
        cli.parse_args(["--frobnicate"])


def test_exit_codes(tmp_path, capsys):
    assert cli.main(["--prompt", "1"]) == 1                             # no model
    assert cli.main(["--model", str(tmp_path / "nope"), "--prompt", "1"]) == 1
    assert cli.main(["--model", str(tmp_path)]) == 1                    # no prompt and no --bench
    assert cli.main(["--model", str(tmp_path), "--prompt", "1", "--backend", "cuda"]) == 1
    assert cli.main(["--help"]) == 0
    assert "--repeat-penalty" in capsys.readouterr().err


def test_prompts(tmp_path):
    assert cli.parse_prompts("1 2 3", ".") == [[1, 2, 3]]
    assert cli.parse_prompts("1,2; 3 4 ;5", ".") == [[1, 2], [3, 4], [5]]
    f = tmp_path / "p.txt"
    f.write_text("7 8\n9")
    assert cli.parse_prompts("@" + str(f), ".") == [[7, 8, 9]]
    with pytest.raises(ValueError, match="tokenizer"):
        cli.parse_prompts("hello there", str(tmp_path))


def test_attention_strategy_strings():
    # Daisi.Llogos/Inference/AttentionStrategy.cs:75-100
    assert api.parse_attention("full") == (None, 0)
    assert api.parse_attention("window:128") == (128, 0)
    assert api.parse_attention("sinks:4,60") == (64, 4)
    for bad in ("window:0", "sinks:4", "ring", "sinks:-1,5"):
        with pytest.raises(ValueError):
            api.parse_attention(bad)


def test_random_subcommand_writes_a_model_folder(tmp_path, llogos):
    import json
    import tiny_configs as tc
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(tc.TINY_A))
    out = tmp_path / "model"
    assert cli.main(["random", "--config", str(cfg), "--output-dir", str(out), "--seed", "4"]) == 0
    ck = llogos.Checkpoint(str(out))
    arch = llogos.architecture_of(tc.TINY_A)
    ck.check(llogos.Model(arch.model_spec(arch.read_config(tc.TINY_A))).tensor_specs())
    assert json.load(open(out / "config.json")) == tc.TINY_A
    assert cli.main(["random", "--config", str(tmp_path / "nope.json"), "--output-dir", str(out)]) == 1
    assert cli.main(["random", "--output-dir", str(out)]) == 1


def test_a_library_built_from_other_sources_is_not_loaded(tmp_path, monkeypatch):
    """A kernel library whose stamp does not match the sources is rebuilt before it is loaded,
    and where that cannot be done loading raises; it is never loaded as it is."""
    import importlib
    library = importlib.import_module("daisi-llogos_amd.ops.library")
    fake_dir = tmp_path / "_build"
    fake_dir.mkdir()
    (fake_dir / library.LIB_NAME).write_bytes(b"not a library")
    (fake_dir / "sources.sha256").write_text("0" * 64)
    monkeypatch.setattr(library, "build_dirs", lambda: [str(fake_dir)])
    monkeypatch.setattr(library, "_PKG", str(tmp_path))
    monkeypatch.setattr(library, "_lib", None)
    monkeypatch.delenv("LLOGOS_KERNEL_LIBRARY", raising=False)
    assert library.is_stale(str(fake_dir / library.LIB_NAME))
    calls = []

    def no_compiler():
        calls.append(1)
        raise library.KernelLibraryError("hipcc not found")
    monkeypatch.setattr(library, "_hipcc", no_compiler)
    import pytest
    with pytest.raises(library.KernelLibraryError, match="stale and cannot be rebuilt"):
        library.load()
    assert calls == [1]
    # a fresh stamp: found and taken as it is (loading these bytes then fails as a load error)
    (fake_dir / "sources.sha256").write_text(library._source_hash())
    assert not library.is_stale(str(fake_dir / library.LIB_NAME))
    with pytest.raises(library.KernelLibraryError, match="cannot load"):
        library.load()
    assert calls == [1]


def test_fractions_of_peak_are_zero_for_a_gpu_without_published_peaks():
    r = api.BenchmarkResult(100, 50, 0.1, 0.5, prefill_flops=1e12, decode_bytes=1e9, peaks={})
    assert r.prefill_fraction_of_peak == 0.0 and r.decode_fraction_of_peak == 0.0
    assert r.decode_bytes_per_second == 2e9 and r.prefill_tokens_per_second == 1000
    known = api.BenchmarkResult(100, 50, 0.1, 0.5, prefill_flops=1e12, decode_bytes=1e9, peaks=api.DEVICE_PEAKS["gfx950"])
    assert known.decode_fraction_of_peak == 2e9 / 8e12 and known.prefill_fraction_of_peak == 1e13 / 2.5e15
    assert api.device_peaks() == {} or "hbm" in api.device_peaks()      # no GPU here: nothing is assumed
