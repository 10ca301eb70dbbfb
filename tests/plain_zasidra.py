"""A plain, slow implementation of the Zasidra decoder: whole sequences, no cache, NumPy float64,
one function for each mechanism.  It shares no code with the package under test: config.json is
read with ``json``, the weights with the ``safetensors`` library.

The design in short (x is the residual stream [T, width], positions p count from 0):

    x = E[token] * embedding scale
    per layer:  x = x + N1(mixer(x));   x = x + N2(ff(x))       the norm stands on the sublayer's output
    logits = W_head N_final(x)

N(y) = y / sqrt(mean(y^2) + eps) * (1 + w).  Mixers: grouped-query attention with an RMS norm over the
whole of q and of k, a partial rotation of split halves with YaRN-stretched frequencies, and a learned
sink in the softmax (`attention`; a layer may read an earlier layer's keys and values instead of
making its own), and attention through a low-rank latent without positions, with a sigmoid gate on every
head's output (`latent_attention`).  Feed-forwards: SwiGLU, or a mixture of SwiGLU experts whose router
adds a correction to its softmax scores for the choice alone, picks within the best groups of
neighbouring experts, counts some router outputs as experts that return their input, and has a shared
expert beside it.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------

def unit_rows(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """The layers' norm: the stored weight is the distance from one."""
    return unit_rows(x, eps) * (1.0 + np.asarray(w, dtype=np.float64))


def plain_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return unit_rows(x, eps) * np.asarray(w, dtype=np.float64)


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-np.asarray(z, dtype=np.float64)))


def silu(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.float64)
    return z * sigmoid(z)


def rotation_frequencies(dims: int, base: float, scaling: dict = None):
    """(frequencies of the dims / 2 pairs, what cos and sin are multiplied with)."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return np.array(f), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return np.array(out), 0.1 * math.log(factor) + 1.0


def rotate_split_halves(x: np.ndarray, positions: np.ndarray, dims: int, freqs: np.ndarray, amplitude: float) -> np.ndarray:
    """x [T, heads, dim]: dimension i of the first `dims` is paired with dimension i + dims / 2; the rest pass."""
    x = np.array(x, dtype=np.float64)
    half = dims // 2
    angle = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]            # [T, half]
    c, s = (np.cos(angle) * amplitude)[:, None, :], (np.sin(angle) * amplitude)[:, None, :]
    u, v = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = u * c - v * s
    x[..., half:dims] = v * c + u * s
    return x


def causal_softmax(scores: np.ndarray, sink: float = None, first: int = 0) -> np.ndarray:
    """scores [Tq, Tk]; query row i stands at position first + i and sees keys 0 .. first + i.  With `sink`
    the denominator also holds exp(sink), which has no column."""
    Tq, Tk = scores.shape
    out = np.zeros_like(scores)
    for i in range(Tq):
        n = first + i + 1
        row = scores[i, :n]
        m = row.max() if sink is None else max(row.max(), sink)
        e = np.exp(row - m)
        den = e.sum() + (math.exp(sink - m) if sink is not None else 0.0)
        out[i, :n] = e / den
    return out


def attention_keys_values(h, t, m: dict, eps: float, positions):
    """The keys (normed over the whole projection, rotated) [T, G, dim] and values [T, G, vdim] of a layer."""
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    k = plain_norm(h @ t["k"].T, t["k.norm"], eps).reshape(T, G, d)
    v = (h @ t["v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot:
        f, amp = rotation_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate_split_halves(k, positions, rot["dims"], f, amp)
    return k, v


def attention(h, t, m: dict, eps: float, positions, keys_values=None):
    """Grouped-query attention.  keys_values: another layer's (k, v) to read instead of this layer's own.
    Returns (output [T, width], (k, v))."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = plain_norm(h @ t["q"].T, t["q.norm"], eps).reshape(T, H, d)
    rot = m.get("rot")
    if rot:
        f, amp = rotation_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate_split_halves(q, positions, rot["dims"], f, amp)
    k, v = keys_values if keys_values is not None else attention_keys_values(h, t, m, eps, positions)
    first = k.shape[0] - T
    out = np.zeros((T, H, dv))
    for head in range(H):
        g = head // (H // G)
        p = causal_softmax((q[:, head] @ k[:, g].T) * m["scale"], float(t["sink"][head]), first)
        out[:, head] = p @ v[:, g]
    return out.reshape(T, H * dv) @ t["o"].T, (k, v)


def latent_attention(h, t, m: dict, eps: float):
    """Attention whose keys and values are both made from one normed latent a token; no positions."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ t["q"].T).reshape(T, H, d)
    c = plain_norm(h @ t["dkv"].T, t["dkv.norm"], eps)                       # [T, rank]
    k = (c @ t["uk"].T).reshape(T, H, d)
    v = (c @ t["uv"].T).reshape(T, H, dv)
    gate = sigmoid(h @ t["g"].T)                                            # [T, H]
    out = np.zeros((T, H, dv))
    for head in range(H):
        p = causal_softmax((q[:, head] @ k[:, head].T) * m["scale"])
        out[:, head] = (p @ v[:, head]) * gate[:, head:head + 1]
    return out.reshape(T, H * dv) @ t["o"].T


def gated_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h, router_w, correction, r: dict):
    """(chosen [T, top] router outputs, weights [T, top]) of each row of h."""
    n = r["experts"] + r.get("identity", 0)
    z = np.asarray(h, dtype=np.float64) @ np.asarray(router_w, dtype=np.float64).T
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    choice = s + np.asarray(correction, dtype=np.float64)[None, :]
    groups = r.get("groups")
    if groups:
        size = n // groups["count"]
        best = choice.reshape(-1, groups["count"], size).max(axis=2)            # [T, groups]
        for row in range(choice.shape[0]):
            kept = np.argsort(-best[row], kind="stable")[:groups["keep"]]
            for g in range(groups["count"]):
                if g not in kept:
                    choice[row, g * size:(g + 1) * size] = -np.inf
    chosen = np.argsort(-choice, axis=1, kind="stable")[:, :r["top"]]
    picked = np.take_along_axis(s, chosen, axis=1)
    weights = picked / (picked.sum(axis=1, keepdims=True) + 1e-20) * r["scale"]
    return chosen, weights


def mixture(h, t, mlp: dict):
    r = mlp["router"]
    chosen, weights = route(h, t["router"], t["correction"], r)
    out = np.zeros_like(np.asarray(h, dtype=np.float64))
    for row in range(h.shape[0]):
        for e, w in zip(chosen[row], weights[row]):
            if e >= r["experts"]:
                out[row] += w * h[row]                                      # an expert that returns its input
            else:
                out[row] += w * gated_ff(h[row:row + 1], t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"])[0]
    if mlp.get("shared"):
        out += gated_ff(h, t["shared.gate"], t["shared.up"], t["shared.down"])
    return out


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------

def load(folder: str):
    """(config dict, {name: float64 array}) of a model folder."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(torch.float64).numpy()
    return cfg, tensors


def part(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: dict, tokens, streams: list = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence.  streams: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = tensors["embed"][np.asarray(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    positions = np.arange(len(tokens))
    kept = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        if L["type"] == "attention":
            src = m.get("kv_from")
            a, kv = attention(x, part(tensors, p + "mix."), m, eps, positions, kept[src] if src is not None else None)
            kept[i] = kv
        elif L["type"] == "latent_attention":
            a = latent_attention(x, part(tensors, p + "mix."), m, eps)
        else:
            raise ValueError(f"unknown layer type {L['type']}")
        x = x + offset_norm(a, tensors[p + "norm1"], eps)
        mlp = L.get("mlp")
        if mlp:
            t = part(tensors, p + "mlp.")
            d = gated_ff(x, t["gate"], t["up"], t["down"]) if mlp["kind"] == "dense" else mixture(x, t, mlp)
            x = x + offset_norm(d, tensors[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.copy())
    return offset_norm(x, tensors["final.norm"], eps) @ tensors["head"].T


def generate_greedy(cfg: dict, tensors: dict, prompt, n: int) -> list:
    """n tokens, each the first largest logit after everything before it (the whole sequence is run again each time)."""
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(np.argmax(forward(cfg, tensors, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
