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
    """Numbers worked out by hand for Llama-3.1-8B, not by the bench's formula."""
    cfg = bench.LLAMA31_8B
    # a layer: qkv 6144 x 4096 = 25,165,824; o 16,777,216; gate, up, down 3 x 58,720,256; two norms 8,192
    # -> 218,112,000 parameters; 32 layers 6,979,584,000; head 128256 x 4096 = 525,336,576; final norm 4,096
    assert bench.weight_bytes(cfg) == 15_009_849_344
    assert bench.kv_bytes_per_token(cfg) == 131_072            # 32 layers x (k + v) x 8 heads x 128 x 2 bytes
    # 2,048 tokens: matrices 2 x 6,979,321,856 x 2048 = 28,587,302,322,176; attention (qk^T and pv, half the
    # square each) 32 x 2 x 4096 x 2048^2 = 1,099,511,627,776; head on one row 1,050,673,152
    assert bench.prefill_flops(cfg, 2048) == 28_587_302_322_176 + 1_099_511_627_776 + 1_050_673_152
    assert bench.HBM_PEAK == 8.0e12 and bench.MFMA_PEAK["bf16"] == 2.5e15 and bench.MFMA_PEAK["fp32"] == 157.3e12
    assert bench.MODELS["llama-3.1-70b"][1]["num_hidden_layers"] == 80 and bench.MODELS["qwen3-14b"][1]["hidden_size"] == 5120


def test_more_than_one_gpu_is_refused_with_one_line():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "4"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "one GPU" in p.stdout
