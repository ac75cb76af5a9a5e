"""Shared by the GPU tests: model folders of the tiny configurations, the plain
implementation's logits, tolerances."""
import functools
import importlib
import os
import tempfile

import numpy as np

import plain_model as pm
import tiny_configs as tc

llogos = importlib.import_module("daisi-llogos_amd")

# float32: the engine against float64 arithmetic, absolute.  bfloat16: the engine's distance from
# float64 arithmetic is set by where values are rounded to bfloat16 (normed rows, rotated
# queries and keys, values, probabilities, the attention's output, the gate/up product,
# silu(gate) * up), so the bound is the distance of the plain implementation with those
# roundings from the plain implementation without them, measured per configuration on a few
# sequences, with a margin of a half (`tol`, `forward_with_roundings`).
TOL = {"float32": 1e-4}
BF16_MARGIN = 1.5
DTYPES = ["float32", "bfloat16"]

_tmp = tempfile.TemporaryDirectory(prefix="llogos_test_models_")


PEAKY = "_peaky"            # suffix of a configuration's name: the same model with sharp attention
PEAKY_FACTOR = 12.0


@functools.lru_cache(maxsize=None)
def folder(name: str, seed: int = 11) -> str:
    """The model folder of a tiny configuration.  `<name>_peaky` is the same model with its query
    and key projections (and their biases) scaled up, so that scores spread over tens of units and
    each query looks at a few keys: a key that is dropped, or one too many, then moves the logits
    by far more than rounding does."""
    path = os.path.join(_tmp.name, f"{name}_{seed}")
    if name.endswith(PEAKY):
        import json
        import shutil
        from safetensors.torch import load_file, save_file
        base = folder(name[:-len(PEAKY)], seed)
        os.makedirs(path, exist_ok=True)
        shutil.copy(os.path.join(base, "config.json"), os.path.join(path, "config.json"))
        tensors = load_file(os.path.join(base, "model.safetensors"))
        for k in tensors:
            if ".q_proj." in k or ".k_proj." in k:
                tensors[k] = (tensors[k].float() * PEAKY_FACTOR).to(tensors[k].dtype)
        save_file(tensors, os.path.join(path, "model.safetensors"))
        tc.ALL.setdefault(name, tc.ALL[name[:-len(PEAKY)]])
        return path
    llogos.write_random_model(path, tc.ALL[name], seed=seed)
    return path


@functools.lru_cache(maxsize=None)
def plain(name: str, seed: int = 11):
    return pm.load_folder(folder(name, seed))


@functools.lru_cache(maxsize=None)
def plain_logits(name: str, tokens: tuple, seed: int = 11) -> np.ndarray:
    cfg, w = plain(name, seed)
    return pm.forward(cfg, w, list(tokens))


def tokens(name: str, n: int, seed: int) -> tuple:
    rng = np.random.default_rng(seed)
    return tuple(int(t) for t in rng.integers(0, tc.ALL[name]["vocab_size"], size=n))


def engine(name: str, dtype: str, max_tokens: int = 2048, n_slots: int = 4, seed: int = 11, **options):
    return llogos.Engine.from_folder(folder(name, seed), dtype=dtype, max_tokens=max_tokens, n_slots=n_slots, **options)


def _bf16(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).to(torch.float64).numpy()


def with_roundings(run):
    """run() with the bfloat16 engine's roundings put into the plain implementation's parts:
    normed rows, rotated queries and keys, values, probabilities (not their sum), the
    attention's output, gate and up, silu(gate) * up.  Sums, softmax, norms and the residual
    stream stay in float64."""
    def attention(q, k, v, n_heads, n_kv_heads, head_dim, scale=None, window=0, sinks=0, positions=None):
        q, k, v = _bf16(q), _bf16(k), _bf16(v)
        T, group = q.shape[0], n_heads // n_kv_heads
        pos = np.arange(T) if positions is None else np.asarray(list(positions))
        seen = pos[None, :] <= pos[:, None]
        if window > 0:
            seen &= (pos[None, :] < sinks) | (pos[None, :] > pos[:, None] - window)
        assert seen[3 % T, 0] == pm.visible(int(pos[3 % T]), int(pos[0]), window, sinks)
        out = np.zeros((T, n_heads * head_dim))
        for h in range(n_heads):
            g = h // group
            qh, kh, vh = (m[:, i * head_dim:(i + 1) * head_dim] for m, i in ((q, h), (k, g), (v, g)))
            s = np.where(seen, (qh @ kh.T) * (scale if scale is not None else 1.0 / np.sqrt(head_dim)), -np.inf)
            p = np.exp(s - s.max(1, keepdims=True))
            out[:, h * head_dim:(h + 1) * head_dim] = (_bf16(p) @ vh) / p.sum(1, keepdims=True)
        return _bf16(out)

    def swiglu_mlp(x, wg, wu, wd):
        g, u = _bf16(pm.linear(x, wg)), _bf16(pm.linear(x, wu))
        return pm.linear(_bf16(pm.silu(g) * u), wd)

    saved = pm.rms_norm, pm.attention, pm.swiglu_mlp
    norm = pm.rms_norm
    pm.rms_norm, pm.attention, pm.swiglu_mlp = (lambda x, w_, eps: _bf16(norm(x, w_, eps))), attention, swiglu_mlp
    try:
        return run()
    finally:
        pm.rms_norm, pm.attention, pm.swiglu_mlp = saved


def forward_with_roundings(cfg, w, tokens, window=None, sinks=0):
    return with_roundings(lambda: pm.forward(cfg, w, list(tokens), window=window, sinks=sinks))


BOUND_LENGTHS = (150, 40, 17, 96)


@functools.lru_cache(maxsize=None)
def rounding_distance(name: str, seed: int = 11) -> float:
    """How far bfloat16 roundings alone move this configuration's logits: the largest
    difference over a few sequences between the plain implementation with and without them."""
    cfg, w = plain(name, seed)
    worst = 0.0
    for i, n in enumerate(BOUND_LENGTHS):
        toks = tokens(name, n, 900 + i)
        worst = max(worst, float(np.abs(forward_with_roundings(cfg, w, toks) - plain_logits(name, toks, seed)).max()))
    return worst


def tol(dtype: str, config: str = None, seed: int = 11) -> float:
    if dtype == "float32":
        return TOL["float32"]
    assert config is not None, "a bfloat16 comparison needs the configuration's name for its bound"
    return BF16_MARGIN * rounding_distance(config, seed)


def close(got, want, dtype: str, what: str = "", config: str = None, seed: int = 11):
    """`got` within the bound of `want`: 1e-4 in float32; in bfloat16 one and a half times the
    distance that bfloat16 roundings alone cause in the plain implementation of `config`."""
    got = np.asarray(got, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - want).max()
    bound = tol(dtype, config, seed)
    assert err <= bound, f"{what}: max abs error {err:.3e} > {bound:.2e} ({dtype})"
    return err
