"""bench.py's arithmetic and its refusal of more than one GPU, without a GPU."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


def test_bytes_and_flops_of_the_8b_sizes():
    cfg = bench.LLAMA31_8B
    # 32 layers of (qkv 4096 x 6144, o 4096 x 4096, gate/up/down 3 x 4096 x 14336, two norms) and the head
    per_layer = 4096 * 6144 + 4096 * 4096 + 3 * 4096 * 14336 + 2 * 4096
    assert bench.weight_bytes(cfg) == (32 * per_layer + 128256 * 4096 + 4096) * 2
    assert abs(bench.weight_bytes(cfg) / 1e9 - 15.0) < 0.05
    assert bench.kv_bytes_per_token(cfg) == 32 * 2 * 8 * 128 * 2 == 131072
    t = 2048
    linear = 32 * (4096 * 6144 + 4096 * 4096 + 3 * 4096 * 14336)
    assert bench.prefill_flops(cfg, t) == 2 * linear * t + 32 * 2 * 4096 * t * t + 2 * 128256 * 4096
    assert bench.HBM_PEAK == 8.0e12 and bench.MFMA_PEAK["bf16"] == 2.5e15 and bench.MFMA_PEAK["fp32"] == 157.3e12
    assert bench.MODELS["llama-3.1-70b"][1]["num_hidden_layers"] == 80 and bench.MODELS["qwen3-14b"][1]["hidden_size"] == 5120


def test_more_than_one_gpu_is_refused_with_one_line():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "4"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
