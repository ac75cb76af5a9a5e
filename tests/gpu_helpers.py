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

# float32: the engine against float64 arithmetic, absolute.  bfloat16: matrices, activations
# and cache rounded to 8 bits of mantissa with all sums in float32; each rounding is a relative
# error of up to 2^-9, so the bound is relative to the size of the logits (of order 1 in the
# tiny models, about 6 at the 8B layer sizes)
TOL = {"float32": 1e-4, "bfloat16": 3e-2}
DTYPES = ["float32", "bfloat16"]

_tmp = tempfile.TemporaryDirectory(prefix="llogos_test_models_")


@functools.lru_cache(maxsize=None)
def folder(name: str, seed: int = 11) -> str:
    path = os.path.join(_tmp.name, f"{name}_{seed}")
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


def close(got, want, dtype: str, what: str = ""):
    got = np.asarray(got, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - want).max()
    tol = TOL[dtype] * (max(1.0, np.abs(want).max()) if dtype == "bfloat16" else 1.0)
    assert err <= tol, f"{what}: max abs error {err:.3e} > {tol:.1e} ({dtype})"
    return err
