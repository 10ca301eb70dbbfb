"""Grouped-query attention over the paged cache.

Order inside the mixer (reference: Daisi.Llogos/Inference/ForwardPass.cs:329-405):
projections q, k, v (:368-370) with their optional biases (:379-382; a bias is part of its
projection here), optional per-head RMSNorm of q and k with one weight per projection
(:372-376), rotation (:385), cache write (:388), attention with kv head = head / group and
scale 1/sqrt(head_dim) after the dot (:336, :391-401), output projection (:404).
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Sequence

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Residual, Runtime, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear
from .rope import Rotary


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True
    takes_normed_rows = True       # h goes into the q/k/v product alone
    adds_to_residual = True        # the output projection can add itself to the stream

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: Rotary, bias: bool = False, qk_norm: bool = False, eps: float = 1e-6,
                 window: int = 0, sinks: int = 0, scale: Optional[float] = None,
                 v_dim: Optional[int] = None, unit_qk: bool = False,
                 names: Sequence[str] = ("q_proj", "k_proj", "v_proj", "o_proj"), suffix: str = ".weight"):
        """v_dim: width of a head's values when it is not head_dim.  unit_qk: after the rotation every head's
        query and key are divided by their root mean square (eps inside the root, no weight).  names, suffix:
        the four matrices' tensor names behind `prefix`.  With either of the first two the step goes through
        the preparation kernel for any head shape (ops.kernels.rotary_prepare) instead of the dense decoder's."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        self.v_dim = int(v_dim) if v_dim else int(head_dim)
        self.unit_qk = bool(unit_qk)
        self.general = self.unit_qk or self.v_dim != head_dim or head_dim % 16 != 0 or position is None
        if self.general:
            if max(head_dim, self.v_dim) > K.GENERIC_MAX_HEAD_DIM:
                raise ValueError(f"heads of {head_dim} and {self.v_dim} dimensions are wider than the attention kernels take")
            if bias or qk_norm:
                raise ValueError("biases and the norm before the rotation are not built beside unit-length queries or values of their own width")
        elif head_dim % 16 or head_dim > K.MAX_HEAD_DIM:
            raise ValueError(f"head_dim {head_dim} must be a multiple of 16, at most {K.MAX_HEAD_DIM}")
        self.prefix = prefix
        self.hidden = hidden
        self.n_heads, self.n_kv_heads, self.head_dim = n_heads, n_kv_heads, head_dim
        self.position = position
        self.qk_norm = qk_norm
        self.eps = float(eps)
        self.window, self.sinks = int(window), int(sinks)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        q_w, kv_w = n_heads * head_dim, n_kv_heads * head_dim
        self.qkv = Linear([prefix + n for n in names[:3]], hidden, [q_w, kv_w, n_kv_heads * self.v_dim], bias=bias, suffix=suffix)
        self.o = Linear([prefix + names[3]], n_heads * self.v_dim, [hidden], suffix=suffix)
        self.q_norm_w: Optional[torch.Tensor] = None
        self.k_norm_w: Optional[torch.Tensor] = None
        self.fuse_decode = True     # single-token steps: one kernel from the projection to the attention output

    def kv_spec(self) -> KVSpec:
        if self.general:         # a head's rows in the pages: its sizes rounded up to the pages' step
            up = lambda n: -(-n // K.HEAD_DIM_STEP) * K.HEAD_DIM_STEP
            return KVSpec(self.n_kv_heads, up(self.head_dim), self.window, self.sinks, v_dim=up(self.v_dim))
        return KVSpec(self.n_kv_heads, self.head_dim, self.window, self.sinks)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.qkv.tensor_specs() + self.o.tensor_specs()
        if self.qk_norm:
            specs.append(TensorSpec(self.prefix + "q_norm.weight", (self.head_dim,), "norm"))
            specs.append(TensorSpec(self.prefix + "k_norm.weight", (self.head_dim,), "norm"))
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.qkv.bind(get, rt)
        self.o.bind(get, rt)
        if self.qk_norm:
            self.q_norm_w = get(self.prefix + "q_norm.weight").to(device=rt.device, dtype=torch.float32).contiguous()
            self.k_norm_w = get(self.prefix + "k_norm.weight").to(device=rt.device, dtype=torch.float32).contiguous()
        if self.position is not None and getattr(self.position, "inv_freq", None) is None:
            self.position.bind(get, rt)

    def forward(self, ctx: StepContext, h, cache: LayerCache, residual: Optional[Residual] = None):
        nh, nkv, hd = self.n_heads, self.n_kv_heads, self.head_dim
        cs = self.position.prepare(ctx) if self.position is not None else None
        if self.general:
            return self._forward_general(ctx, h, cache, cs, residual)
        if cache.writes:
            qkv = self.qkv.product(h, f32_ok=True)                      # [(parts,) T, (nh + 2 nkv) hd]
            mark(ctx, "qkv")
            if ctx.is_decode and self.fuse_decode:
                # one token a sequence: norm, rotation and cache write inside the attention kernel
                a = K.attention_decode_fused(ctx, qkv, self.qkv.bias_rows(), nh, nkv, hd, self.position.rot,
                                             self.position.pairing, self.q_norm_w, self.k_norm_w, self.eps, cs,
                                             cache.k_pool, cache.v_pool, cache.table, self.scale, self.window,
                                             self.sinks)
                if a is not None:
                    mark(ctx, "attention")
                    return self._project(ctx, a, residual)
            q = K.qk_rope_cache(qkv, self.qkv.bias_rows(), self.rt.dtype, nh, nkv, hd, self.position.rot,
                                self.position.pairing, self.q_norm_w, self.k_norm_w, self.eps, cs,
                                cache.k_pool, cache.v_pool, cache.table, ctx.tok_seq, ctx.tok_pos)
        else:
            # the keys and values of these positions are another layer's: project q alone
            qkv = self.qkv.product(h, rows_out=nh * hd, f32_ok=True)
            mark(ctx, "qkv")
            q = K.qk_rope_cache(qkv, self.qkv.bias_rows(nh * hd), self.rt.dtype, nh, 0, hd, self.position.rot,
                                self.position.pairing, self.q_norm_w, None, self.eps, cs, None, None, None,
                                ctx.tok_seq, ctx.tok_pos)
        mark(ctx, "rotation")
        a = K.attention(ctx, q, q.stride(0), cache.k_pool, cache.v_pool, cache.table,
                        nh, nkv, hd, self.scale, self.window, self.sinks)
        mark(ctx, "attention")
        return self._project(ctx, a, residual)

    def _forward_general(self, ctx: StepContext, h, cache: LayerCache, cs: torch.Tensor, residual: Optional[Residual]):
        """Heads whose queries and keys are made unit length behind the rotation, or whose values have a width of
        their own: preparation for any head shape, then the matrix-core attention where the cache's rows are ones
        it takes, else the kernel for any shape."""
        nh, nkv, hd, vd = self.n_heads, self.n_kv_heads, self.head_dim, self.v_dim
        rows = self.qkv.product(h, f32_ok=True) if cache.writes else self.qkv.product(h, rows_out=nh * hd, f32_ok=True)
        mark(ctx, "qkv")
        rot, pairing = (self.position.rot, self.position.pairing) if self.position is not None else (0, 0)
        q = K.rotary_prepare(ctx, rows, None, self.rt.dtype, nh, nkv, hd, vd, 1, rot, pairing, cs,
                             None, None, self.unit_qk, self.eps, cache.k_pool, cache.v_pool, cache.table, writes=cache.writes)
        mark(ctx, "rotation")
        spec = self.kv_spec()
        if vd == hd and spec.head_dim == hd:
            a = K.attention(ctx, q, q.stride(0), cache.k_pool, cache.v_pool, cache.table, nh, nkv, hd, self.scale,
                            self.window, self.sinks)
        else:
            a = K.attention_generic(q, q.stride(0), cache.k_pool, cache.v_pool, cache.table, ctx.tok_seq, ctx.tok_pos,
                                    nh, nkv, hd, self.scale, self.window, self.sinks, v_dim=vd)
        mark(ctx, "attention")
        return self._project(ctx, a, residual)

    def _project(self, ctx: StepContext, a: torch.Tensor, residual: Optional[Residual] = None):
        out = self.o.add_to(a, residual) if residual is not None else None
        if out is None:
            out = self.o.product(a, f32_ok=True)    # the residual sum that follows adds the parts
        mark(ctx, "o")
        return out
