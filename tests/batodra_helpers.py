"""Shared by the Batodra tests: model folders of the small configurations (random weights, with the query
and key matrices of the attentions scaled up so that attention is sharp and a lost or extra key, a lost first
token or a wrong position shows, and the recurrence's decay spread so that some channels remember hundreds
of tokens), the plain implementation's logits, and the bounds."""
import functools
import importlib
import os
import tempfile

import numpy as np

import batodra_configs as bc
import plain_batodra as pb

llogos = importlib.import_module("daisi-llogos_amd")
_tmp = tempfile.TemporaryDirectory(prefix="llogos_test_batodra_")
DTYPES = ["float32", "bfloat16"]
# float32: the engine against float64 arithmetic, relative to the largest logit.  bfloat16: rounding of the
# matrix products' inputs; the bound is loose, and what must not happen (a key too few, a lost state) is
# asserted in float32 and, with a margin, on sharpened models.
TOL = {"float32": 2e-4, "bfloat16": 0.12}


@functools.lru_cache(maxsize=None)
def folder(name: str, seed: int = 5) -> str:
    from safetensors.torch import load_file, save_file
    path = os.path.join(_tmp.name, f"{name}_{seed}")
    llogos.write_random_model(path, bc.ALL[name], seed=seed, std=0.08)
    file = os.path.join(path, "model.safetensors")
    tensors = load_file(file)
    for k in tensors:
        if k.endswith((".mix.q", ".mix.k")):
            tensors[k] = (tensors[k].float() * 3.0).to(tensors[k].dtype)
        if k.endswith((".mix.q.norm", ".mix.k.norm")):
            tensors[k] = (tensors[k].float() * 1.5).to(tensors[k].dtype)
        if k.endswith((".mix.ra", ".mix.ri", ".mix.x", ".mix.y")):
            tensors[k] = (tensors[k].float() * 4.0).to(tensors[k].dtype)
        if k.endswith(".mix.lam"):                              # decays from a token or two to hundreds of tokens
            t = tensors[k].float()
            tensors[k] = (t * 4.0 - 5.0).to(tensors[k].dtype)
        if k.endswith((".lq1", ".lk1", ".lq2", ".lk2")):
            tensors[k] = (tensors[k].float() * 5.0).to(tensors[k].dtype)
    save_file(tensors, file)
    return path


@functools.lru_cache(maxsize=None)
def plain(name: str, seed: int = 5):
    return pb.load_folder(folder(name, seed))


@functools.lru_cache(maxsize=None)
def plain_logits(name: str, tokens: tuple, seed: int = 5) -> np.ndarray:
    cfg, w = plain(name, seed)
    return pb.forward(cfg, w, list(tokens))


def tokens(name: str, n: int, seed: int) -> tuple:
    rng = np.random.default_rng(seed)
    return tuple(int(t) for t in rng.integers(0, bc.ALL[name]["vocab"], size=n))


def engine(name: str, dtype: str, max_tokens: int = 1024, n_slots: int = 4, seed: int = 5, **options):
    return llogos.Engine.from_folder(folder(name, seed), dtype=dtype, max_tokens=max_tokens, n_slots=n_slots, **options)


def distance(got, want) -> float:
    """Largest difference of the logits, relative to the largest logit's size."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), "not finite"
    return float(np.abs(got - want).max() / max(1e-9, np.abs(want).max()))


def close(got, want, dtype: str, what: str = "") -> float:
    d = distance(got, want)
    assert d <= TOL[dtype], f"{what}: relative error {d:.3e} > {TOL[dtype]:.1e} ({dtype})"
    return d
