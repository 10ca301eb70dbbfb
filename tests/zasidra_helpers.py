"""Shared by the Zasidra tests: model folders of the small configurations (random weights, with the query
and key matrices scaled up so that attention is sharp and a lost or extra key, a lost sink or a wrong
position shows), the plain implementation's logits, and the bounds.

Every model comes in two forms.  In the first the router's choice follows the input: a token whose two
best candidates lie closer than rounding moves them changes its experts, which in 32-bit happens about
never and in bfloat16 (a stream that is a hundredth off) to a token in a hundred, whose logits and all
later ones then have nothing to do with the plain result.  The float32 tests use that form.  The
bfloat16 tests of whole models use the second, in which the corrections lie two units apart, so that they
alone decide the choice (the same outputs for every token; the scores still make the weights); that
bfloat16 follows the same rules for the choice is tested on the feed-forward alone, row by row."""
import functools
import importlib
import os
import tempfile

import numpy as np
import torch

import plain_zasidra as pz
import zasidra_configs as zc

llogos = importlib.import_module("daisi-llogos_amd")
_tmp = tempfile.TemporaryDirectory(prefix="llogos_test_zasidra_")
DTYPES = ["float32", "bfloat16"]
# float32: the engine against float64 arithmetic, relative to the largest logit.  bfloat16: rounding of the
# matrix products' inputs; the bound is loose, and what must not happen (a key too few, a lost sink) is
# asserted in float32 and, with a margin, on sharpened models.
TOL = {"float32": 2e-4, "bfloat16": 0.12}


def sharpen(tensors: dict, fixed_choice: bool = False) -> dict:
    """The weights of the norms over q and k scaled up (the matrices before those norms do not set the scores' size), the
    latent layers' key matrices too.  fixed_choice: corrections two units apart."""
    for k in sorted(tensors):
        t = tensors[k]
        if fixed_choice and k.endswith(".mlp.correction"):
            order = np.random.default_rng(len(k) * 1000 + t.numel() + int(k[1:k.index(".")])).permutation(t.numel())
            tensors[k] = (t.float() * 0 + 2.0 * torch.tensor(order)).to(t.dtype)
        if k.endswith(".mix.uk"):                               # (the latent layers' scores grow with the stream as it is)
            tensors[k] = (t.float() * 1.5).to(t.dtype)
        if k.endswith((".mix.q.norm", ".mix.k.norm")):
            tensors[k] = (t.float() * 1.6).to(t.dtype)
        if k.endswith(".mix.sink"):                             # sinks that weigh as much as the best keys
            tensors[k] = (t.float() * 2.0 + 1.0).to(t.dtype)
    return tensors


def fixed_choice(dtype: str) -> bool:
    return dtype == "bfloat16"


@functools.lru_cache(maxsize=None)
def folder(name: str, seed: int = 5, dtype: str = "float32") -> str:
    from safetensors.torch import load_file, save_file
    path = os.path.join(_tmp.name, f"{name}_{seed}_{'fixed' if fixed_choice(dtype) else 'free'}")
    llogos.write_random_model(path, zc.ALL[name], seed=seed, std=0.08)
    file = os.path.join(path, "model.safetensors")
    save_file(sharpen(load_file(file), fixed_choice(dtype)), file)
    return path


@functools.lru_cache(maxsize=None)
def plain(name: str, seed: int = 5, dtype: str = "float32"):
    return pz.load(folder(name, seed, dtype))


@functools.lru_cache(maxsize=None)
def plain_logits(name: str, tokens: tuple, seed: int = 5, dtype: str = "float32") -> np.ndarray:
    cfg, w = plain(name, seed, dtype)
    return pz.forward(cfg, w, list(tokens))


def tokens(name: str, n: int, seed: int) -> tuple:
    rng = np.random.default_rng(seed)
    return tuple(int(t) for t in rng.integers(0, zc.ALL[name]["vocab"], size=n))


def engine(name: str, dtype: str, max_tokens: int = 1024, n_slots: int = 4, seed: int = 5, **options):
    return llogos.Engine.from_folder(folder(name, seed, dtype), dtype=dtype, max_tokens=max_tokens, n_slots=n_slots, **options)


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
