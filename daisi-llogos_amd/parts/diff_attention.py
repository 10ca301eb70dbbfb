"""Differential attention: every head has two score maps over the same values, and its output is their
weighted difference, normed.

    q = W_q h   [heads x (map 1 | map 2) x dim],   k = W_k h   [kv_heads x (map 1 | map 2) x dim],   v = W_v h   [kv_heads x v_dim]
    every run of dim values of q and k: RMS norm with a weight shared by all runs of q (of k), then the rotation
    a_m = softmax_j((q_m(i) . k_m(j)) * scale) v(j),  j <= i               m = 1, 2
    lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff                           one number for the layer
    o   = a_1 - lam * a_2;   out = W_o [o / sqrt(mean(o^2) + eps) * (1 - diff)]_heads

Query head h reads key/value head h // (heads / kv_heads).  A kv head's key row in the cache holds both maps' keys
side by side, so one page walk serves both maps and the values are read once.  `lam` is worked out once, in
float32, when the tensors are bound."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Runtime, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear
from .rope import Rotary

MAPS = 2


def _page_row(n: int) -> int:
    return -(-n // K.HEAD_DIM_STEP) * K.HEAD_DIM_STEP


@register_mixer("diff_attention")
class DiffAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, v_dim: int, scale: float,
                 diff: float, position: Optional[Rotary], eps: float = 1e-6, window: int = 0, sinks: int = 0):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if MAPS * head_dim > K.GENERIC_MAX_HEAD_DIM or v_dim > K.GENERIC_MAX_HEAD_DIM:
            raise ValueError(f"heads of 2 x {head_dim} and {v_dim} dimensions are wider than the attention kernels take")
        self.prefix, self.hidden = prefix, int(hidden)
        self.n_heads, self.n_kv_heads, self.head_dim, self.v_dim = int(n_heads), int(n_kv_heads), int(head_dim), int(v_dim)
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.window, self.sinks = int(window), int(sinks)
        self.position = position
        self.qkv = Linear([prefix + "q", prefix + "k", prefix + "v"], hidden,
                          [self.n_heads * MAPS * self.head_dim, self.n_kv_heads * MAPS * self.head_dim, self.n_kv_heads * self.v_dim], suffix="")
        self.o = Linear([prefix + "o"], self.n_heads * self.v_dim, [hidden], suffix="")
        self.q_norm_w = self.k_norm_w = None
        self.lam = 0.0

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.n_kv_heads, _page_row(MAPS * self.head_dim), self.window, self.sinks, v_dim=_page_row(self.v_dim))

    def tensor_specs(self) -> List[TensorSpec]:
        p, d = self.prefix, self.head_dim
        return self.qkv.tensor_specs() + [TensorSpec(p + "q.norm", (d,), "norm"), TensorSpec(p + "k.norm", (d,), "norm")] + \
            [TensorSpec(p + n, (d,), "bias") for n in ("lq1", "lk1", "lq2", "lk2")] + self.o.tensor_specs()

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.qkv.bind(get, rt)
        self.o.bind(get, rt)
        f32 = lambda name: get(self.prefix + name).to(device=rt.device, dtype=torch.float32).contiguous()
        self.q_norm_w, self.k_norm_w = f32("q.norm"), f32("k.norm")
        host = lambda name: get(self.prefix + name).to(device="cpu", dtype=torch.float32)
        self.lam = float(torch.exp((host("lq1") * host("lk1")).sum()) - torch.exp((host("lq2") * host("lk2")).sum())) + self.diff
        if self.position is not None and getattr(self.position, "inv_freq", None) is None:
            self.position.bind(get, rt)

    def forward(self, ctx: StepContext, h, cache: LayerCache):
        nh, nkv, d, vd = self.n_heads, self.n_kv_heads, self.head_dim, self.v_dim
        cs = self.position.prepare(ctx) if self.position is not None else None
        rot, pairing = (self.position.rot, self.position.pairing) if self.position is not None else (0, 0)
        rows = self.qkv.product(h, f32_ok=True) if cache.writes else self.qkv.product(h, rows_out=nh * MAPS * d, f32_ok=True)
        mark(ctx, "qkv")
        q = K.rotary_prepare(ctx, rows, None, self.rt.dtype, nh, nkv, d, vd, MAPS, rot, pairing, cs,
                             self.q_norm_w, self.k_norm_w, False, self.eps, cache.k_pool, cache.v_pool, cache.table,
                             writes=cache.writes)
        mark(ctx, "rotation")
        a = K.diff_attention(ctx, q, cache.k_pool, cache.v_pool, cache.table, nh, nkv, d, vd, self.scale, self.lam,
                             1.0 - self.diff, self.eps, self.window, self.sinks)
        mark(ctx, "attention")
        out = self.o.product(a, f32_ok=True)
        mark(ctx, "o")
        return out
