"""A plain, slow implementation of the Batodra decoder: whole sequences, no cache, NumPy float64,
one function for each mechanism.  It shares no code with the package under test: config.json is
read with ``json``, the weights with the ``safetensors`` library.

The design in short (x is the residual stream [T, width], positions p count from 0):

    x = E[token]
    per layer:  x = N1(alpha x + mixer(x));   x = N2(alpha x + ff(x))     the norm comes after the sum
    logits = W_head N_final(x)

A layer may borrow another layer's tensors (`weights_of`).  Mixers: a gated linear recurrence
(`rglru`), differential attention with per-head norms before the rotation (`attention`), and attention
over a sliding window that keeps the first tokens, with YaRN-scaled rotation and unit-length queries and
keys (`attention_2`).  The feed-forward is two matrices around the square of relu.
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


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return unit_rows(x, eps) * np.asarray(w, dtype=np.float64)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z: np.ndarray) -> np.ndarray:
    return np.maximum(np.asarray(z, dtype=np.float64), 0.0) ** 2


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-np.asarray(z, dtype=np.float64)))


def softplus(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.float64)
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def time_convolution(u: np.ndarray, taps: np.ndarray, bias: np.ndarray, before: np.ndarray = None) -> np.ndarray:
    """y_t = bias + sum_j taps[:, j] u_(t - n + 1 + j) for n taps a channel: the last column weighs the
    present row.  Rows before the first are `before` ([n - 1, channels], oldest first) or zeros."""
    u, taps = np.asarray(u, dtype=np.float64), np.asarray(taps, dtype=np.float64)
    n = taps.shape[1]
    pad = np.zeros((n - 1, u.shape[1])) if before is None else np.asarray(before, dtype=np.float64)
    full = np.concatenate([pad, u], axis=0)
    out = np.tile(np.asarray(bias, dtype=np.float64), (u.shape[0], 1))
    for t in range(u.shape[0]):
        for j in range(n):
            out[t] += taps[:, j] * full[t + j]
    return out


def block_products(u: np.ndarray, mats: np.ndarray, bias: np.ndarray) -> np.ndarray:
    """u [T, C] cut into len(mats) equal parts; part b goes through its own square matrix mats[b]
    ([out, in]) and gets bias[b]."""
    u = np.asarray(u, dtype=np.float64)
    nb = mats.shape[0]
    size = u.shape[1] // nb
    out = np.zeros_like(u)
    for b in range(nb):
        part = u[:, b * size:(b + 1) * size]
        out[:, b * size:(b + 1) * size] = part @ np.asarray(mats[b], dtype=np.float64).T + np.asarray(bias[b], dtype=np.float64)
    return out


DECAY_SHARPNESS = 8.0


def gated_recurrence(u: np.ndarray, r: np.ndarray, i: np.ndarray, lam: np.ndarray, state: np.ndarray = None):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-8 r_t softplus(lam)); S starts at
    `state` (zeros by default).  Returns (all S_t [T, C], the last S)."""
    u = np.asarray(u, dtype=np.float64)
    S = np.zeros(u.shape[1]) if state is None else np.asarray(state, dtype=np.float64).copy()
    sp = softplus(lam)
    out = np.zeros_like(u)
    for t in range(u.shape[0]):
        a = np.exp(-DECAY_SHARPNESS * r[t] * sp)
        S = a * S + np.sqrt(1.0 - a * a) * i[t] * u[t]
        out[t] = S
    return out, S


def rotary_frequencies(dims: int, base: float, scaling: dict = None):
    """(frequencies [dims / 2], amplitude).  f_i = base^(-2i / dims); with YaRN scaling (factor, original,
    fast, slow) the pairs that turn often keep f_i, those that turn seldom get f_i / factor, with a ramp
    over the pair index between, and cos and sin are stretched by 0.1 ln(factor) + 1."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: np.ndarray, positions, dims: int, freqs: np.ndarray, amplitude: float = 1.0) -> np.ndarray:
    """x [T, n, D]: the first `dims` of the D dimensions are turned, dimension i with i + dims / 2."""
    x = np.asarray(x, dtype=np.float64).copy()
    half = dims // 2
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    c, s = (np.cos(ang) * amplitude)[:, None, :], (np.sin(ang) * amplitude)[:, None, :]
    a, b = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = a * c - b * s
    x[..., half:dims] = b * c + a * s
    return x


def visible(positions, window: int = 0, keep_first: int = 0) -> np.ndarray:
    """[T, T] booleans: query i sees key j when j <= i and, with a window, i - j < window or j < keep_first."""
    p = np.asarray(positions)
    i, j = p[:, None], p[None, :]
    ok = j <= i
    if window > 0:
        ok &= (i - j < window) | (j < keep_first)
    return ok


def softmax_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, mask: np.ndarray) -> np.ndarray:
    """q [T, H, D], k [T, G, D], v [T, G, Dv]: head h reads key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(mask, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, g]
    return out


def difference_weight(lq1, lk1, lq2, lk2, diff: float) -> float:
    f = lambda a, b: math.exp(float(np.sum(np.asarray(a, dtype=np.float64) * np.asarray(b, dtype=np.float64))))
    return f(lq1, lk1) - f(lq2, lk2) + diff


# --------------------------------------------------------------------------
# mixers
# --------------------------------------------------------------------------

def rglru_mixer(m: dict, w: dict, p: str, h: np.ndarray, carry: dict = None) -> np.ndarray:
    """carry: {'conv': the last taps - 1 inputs of the convolution, 'state': S} of the tokens before; it is
    updated in place when given."""
    g = lambda n: np.asarray(w[p + n], dtype=np.float64)
    y = gelu_tanh(h @ g("y").T + g("y.b"))
    xin = h @ g("x").T + g("x.b")
    before = carry.get("conv") if carry is not None else None
    u = time_convolution(xin, g("conv"), g("conv.b"), before)
    r = sigmoid(block_products(u, g("ra"), g("ra.b")))
    i = sigmoid(block_products(u, g("ri"), g("ri.b")))
    S, last = gated_recurrence(u, r, i, g("lam"), carry.get("state") if carry is not None else None)
    if carry is not None:
        n = m["conv"] - 1
        full = xin if before is None else np.concatenate([before, xin], axis=0)
        if full.shape[0] < n:
            full = np.concatenate([np.zeros((n - full.shape[0], xin.shape[1])), full], axis=0)
        carry["conv"] = full[full.shape[0] - n:]
        carry["state"] = last
    return (S * y) @ g("o").T


def differential_attention(m: dict, w: dict, p: str, h: np.ndarray, positions, eps: float) -> np.ndarray:
    g = lambda n: np.asarray(w[p + n], dtype=np.float64)
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ g("q").T).reshape(T, H * 2, D)         # head by head, [map 1, map 2]
    k = (h @ g("k").T).reshape(T, G * 2, D)
    v = (h @ g("v").T).reshape(T, G, Dv)
    q, k = rms_norm(q, g("q.norm"), eps), rms_norm(k, g("k.norm"), eps)
    f, amp = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q, k = rotate(q, positions, m["rot"]["dims"], f, amp), rotate(k, positions, m["rot"]["dims"], f, amp)
    mask = visible(positions)
    q, k = q.reshape(T, H, 2, D), k.reshape(T, G, 2, D)
    a1 = softmax_attention(q[:, :, 0], k[:, :, 0], v, m["scale"], mask)
    a2 = softmax_attention(q[:, :, 1], k[:, :, 1], v, m["scale"], mask)
    lam = difference_weight(g("lq1"), g("lk1"), g("lq2"), g("lk2"), m["diff"])
    o = unit_rows(a1 - lam * a2, eps) * (1.0 - m["diff"])
    return o.reshape(T, H * Dv) @ g("o").T


def window_attention(m: dict, w: dict, p: str, h: np.ndarray, positions, eps: float) -> np.ndarray:
    g = lambda n: np.asarray(w[p + n], dtype=np.float64)
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ g("q").T).reshape(T, H, D)
    k = (h @ g("k").T).reshape(T, G, D)
    v = (h @ g("v").T).reshape(T, G, Dv)
    f, amp = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    q, k = rotate(q, positions, m["rot"]["dims"], f, amp), rotate(k, positions, m["rot"]["dims"], f, amp)
    q, k = unit_rows(q, eps), unit_rows(k, eps)
    mask_cfg = m.get("mask") or {}
    mask = visible(positions, int(mask_cfg.get("size", 0)), int(mask_cfg.get("keep_first", 0)))
    o = softmax_attention(q, k, v, m["scale"], mask)
    return o.reshape(T, H * Dv) @ g("o").T


def feed_forward(w: dict, p: str, h: np.ndarray) -> np.ndarray:
    g = lambda n: np.asarray(w[p + n], dtype=np.float64)
    return relu_squared(h @ g("up").T) @ g("down").T


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------

def load_folder(folder: str):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, {k: v.double().numpy() if v.is_floating_point() else v.numpy() for k, v in tensors.items()}


def forward(cfg: dict, w: dict, tokens, positions=None, streams: list = None, carries: list = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence.  streams: a list that receives the stream after every layer.
    carries: one dict a layer (for the recurrent layers' state), so that a sequence can be continued:
    only models without attention layers can be continued this way (attention needs the whole sequence)."""
    tokens = list(tokens)
    pos = np.arange(len(tokens)) if positions is None else np.asarray(positions)
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = np.asarray(w["embed"], dtype=np.float64)[tokens]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of")
        p = f"l{i if src is None else src}."
        m = layer["mixer"]
        if layer["type"] == "rglru":
            a = rglru_mixer(m, w, p + "mix.", x, carries[i] if carries is not None else None)
        elif layer["type"] == "attention":
            a = differential_attention(m, w, p + "mix.", x, pos, eps)
        elif layer["type"] == "attention_2":
            a = window_attention(m, w, p + "mix.", x, pos, eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']}")
        x = rms_norm(alpha * x + a, w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = rms_norm(alpha * x + feed_forward(w, p + "mlp.", x), w[p + "norm2"], eps)
        if streams is not None:
            streams.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ np.asarray(w["head"], dtype=np.float64).T


def generate_greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    tokens, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(forward(cfg, w, tokens)[-1]))
        out.append(t)
        tokens.append(t)
    return out
