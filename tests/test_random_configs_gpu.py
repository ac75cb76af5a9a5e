"""Configurations drawn at random (fixed seeds) over everything config.json can vary: the
architecture's name and its defaults, head size in steps of 16, heads and groups, widths and
vocabularies that are no power of two, layers, eps, rotary base and scaling, bias, per-head
norm, tied head, windows.  Each runs a ragged prompt step, single-token steps with a sequence
ending early, and a continued prompt, against the plain implementation in both element types:
the kernels take every size the configuration allows, or refuse it; they never give a wrong
result."""
import numpy as np
import pytest

import gpu_helpers as H
import tiny_configs as tc

pytestmark = pytest.mark.gpu
SEEDS = list(range(18)) + [35, 59]      # (35, 59: an output projection over 9 stages of k in 4 parts)


def random_config(seed: int) -> dict:
    rng = np.random.default_rng(1000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    arch = pick(["LlamaForCausalLM", "Qwen2ForCausalLM", "Qwen3ForCausalLM"])
    head_dim = int(pick([16, 32, 48, 64, 80, 96, 112, 128]))
    n_kv = int(pick([1, 2, 3, 4]))
    group = int(pick([1, 2, 3, 4, 5, 8, 16]))
    cfg = {
        "architectures": [arch], "vocab_size": int(pick([97, 256, 331, 1000])), "hidden_size": int(pick([40, 72, 96, 136, 200])),
        "intermediate_size": int(pick([48, 88, 176, 264])), "num_hidden_layers": int(pick([1, 2, 3])),
        "num_attention_heads": n_kv * group, "num_key_value_heads": n_kv, "head_dim": head_dim,
        "rms_norm_eps": float(pick([1e-6, 1e-5, 3e-4])), "rope_theta": float(pick([1e4, 5e5, 1e6])),
        "max_position_embeddings": 4096, "tie_word_embeddings": bool(pick([True, False])),
        "torch_dtype": "bfloat16", "eos_token_id": 1,
    }
    scaling = pick(["none", "llama3", "linear"])
    if scaling == "llama3":
        cfg["rope_scaling"] = {"rope_type": "llama3", "factor": float(pick([4.0, 8.0])), "low_freq_factor": 1.0,
                               "high_freq_factor": 4.0, "original_max_position_embeddings": int(pick([32, 64]))}
    elif scaling == "linear":
        cfg["rope_scaling"] = {"rope_type": "linear", "factor": 2.0}
    if arch == "Qwen2ForCausalLM" and pick([True, False]):
        cfg.update(use_sliding_window=True, sliding_window=int(pick([5, 64, 70, 130])),
                   max_window_layers=int(pick([0, 1])))
    if arch == "LlamaForCausalLM" and pick([True, False]):
        cfg["attention_bias"] = True
    if pick([True, False, False]):
        cfg["partial_rotary_factor"] = 0.5              # the rest of each head is not rotated
    return cfg


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("seed", SEEDS)
def test_random_configuration(seed, dtype):
    name = f"random_{seed}"
    tc.ALL[name] = random_config(seed)
    rng = np.random.default_rng(seed)
    lens = [int(rng.integers(1, 150)) for _ in range(3)]
    seqs = [H.tokens(name, n + 6, 10 * seed + i) for i, n in enumerate(lens)]
    plain = [H.plain_logits(name, s) for s in seqs]
    eng = H.engine(name, dtype, max_tokens=64 * 12, n_slots=3)
    slots = [eng.alloc_slot() for _ in seqs]
    got = eng.step([(sl, s[:n]) for sl, s, n in zip(slots, seqs, lens)], want="all")
    H.close(got.cpu().double().numpy(), np.concatenate([p[:n] for p, n in zip(plain, lens)]), dtype, f"{name}: prompts", config=name)
    live = [0, 1, 2]
    for t in range(4):
        if t == 2:                                      # the second sequence ends early; its slot takes a new prompt later
            eng.free_slot(slots[1])
            live = [0, 2]
        got = eng.step([(slots[i], [seqs[i][lens[i] + t]]) for i in live], want="last")
        H.close(got.cpu().double().numpy(), np.stack([plain[i][lens[i] + t] for i in live]), dtype, f"{name}: token {t}", config=name)
    # a continued prompt of two tokens beside a new prompt in the freed slot
    slots[1] = eng.alloc_slot()
    got = eng.step([(slots[0], seqs[0][lens[0] + 4:lens[0] + 6]), (slots[1], seqs[1][:lens[1]])], want=[[0, 1], [lens[1] - 1]])
    want = np.stack([plain[0][lens[0] + 4], plain[0][lens[0] + 5], plain[1][lens[1] - 1]])
    H.close(got.cpu().double().numpy(), want, dtype, f"{name}: continued prompt beside a new one", config=name)
