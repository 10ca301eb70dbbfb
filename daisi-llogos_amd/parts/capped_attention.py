"""Grouped-query softmax attention with keys and values of different widths, whose every mechanism
beyond the plain softmax is an option: positions through a factor on the query or through a rotation
behind a norm over the whole projection, scores bent through a tanh, a sink in the softmax, a gate on
every head's output.

    [q | k | v | g] = W h (+ biases)                            g: one gate logit a head (optional)
    q, k, v <- conv(q), conv(k), conv(v)                        a short causal convolution over time on every
                                                                channel, directly behind the projection (optional)
    q <- rmsnorm_all(q) * wq;  k <- rmsnorm_all(k) * wk         over the whole projection, all heads at once (optional)
    q, k <- rotate(q), rotate(k)                                the first dimensions of every head, by a position
                                                                encoding's table of cosines and sines (optional)
    q_t <- q_t * (1 + coef * ln(floor((t + 1) / every) + 1))    (optional)
    s(i, j) = cap * tanh((q_i . k_j) * scale / cap),  j <= i    (cap 0: the score as it is)
    p(i, j) = exp(s(i, j)) / (sum_j exp(s(i, j)) [+ exp(z_h)])  a sink without a key or a value: of score 0, or a
                                                                learned score a head (optional)
    out = W_o [sigmoid(g_h) * sum_j p_h(i, j) v_j]_h (+ bias)

Query head h reads key/value head h // (heads / kv_heads).  The convolution's state is the last
taps - 1 projected rows of a sequence, kept for each cache slot beside the pages.  A mixer without keys
and values of its own (own_kv False) has the query's tensors alone and reads the pages that another
layer's run wrote: the model's schedule says whose."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Residual, Runtime, StateSpec, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear
from .rope import Rotary


def _page_row(n: int) -> int:
    """A head's row in the cache's pages: its size rounded up to the pages' step."""
    return -(-n // K.HEAD_DIM_STEP) * K.HEAD_DIM_STEP


@register_mixer("capped_attention")
class CappedAttention(Mixer):
    graph_safe = True
    adds_to_residual = True        # the output projection can add itself to the stream

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, v_dim: int, scale: float,
                 softcap: float = 0.0, temp_coef: float = 0.0, temp_every: int = 1, eps: float = 1e-6, bias: bool = False,
                 unit_sink: bool = False, conv_taps: int = 0, whole_norm: bool = False, head_gate: bool = False,
                 position: Optional[Rotary] = None, learned_sink: bool = False, own_kv: bool = True):
        """position: a rotation of q and k behind their norm (its table of cosines and sines, its rotated width and
        pairing).  learned_sink: the sink's score is the tensor `sink` [heads] (unit_sink: zero).  own_kv False: the
        layer has no key and value tensors (projections, norm) and reads another run's pages."""
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if max(head_dim, v_dim) > K.GENERIC_MAX_HEAD_DIM:
            raise ValueError(f"heads of {head_dim} and {v_dim} dimensions are wider than the attention kernels take ({K.GENERIC_MAX_HEAD_DIM})")
        if conv_taps > K.MAX_CONV_TAPS:
            raise ValueError(f"a convolution of {conv_taps} taps is more than {K.MAX_CONV_TAPS}")
        self.prefix, self.hidden = prefix, int(hidden)
        self.n_heads, self.n_kv_heads, self.head_dim, self.v_dim = int(n_heads), int(n_kv_heads), int(head_dim), int(v_dim)
        self.scale, self.softcap = float(scale), float(softcap)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.eps = float(eps)
        self.has_bias, self.unit_sink, self.conv_taps = bool(bias), bool(unit_sink), int(conv_taps)
        self.whole_norm, self.head_gate = bool(whole_norm), bool(head_gate)
        self.position, self.learned_sink, self.own_kv = position, bool(learned_sink), bool(own_kv)
        if self.learned_sink and self.unit_sink:
            raise ValueError("a sink is of score 0 or learned, not both")
        if position is not None and position.rot > self.head_dim:
            raise ValueError(f"a rotation of {position.rot} dimensions in heads of {self.head_dim}")
        if not self.own_kv and self.conv_taps:
            raise ValueError("a convolution behind the projections needs keys and values of the layer's own")
        self.Wq, self.Wk, self.Wv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim, self.n_kv_heads * self.v_dim
        names, outs = [prefix + "q", prefix + "k", prefix + "v"], [self.Wq, self.Wk, self.Wv]
        if not self.own_kv:
            names, outs = names[:1], outs[:1]
        # the gate reads the same rows as the projections: one product makes all four.  (A gate with a bias
        # would need one for its rows too; this form has none.)
        if self.head_gate and not self.has_bias:
            names.append(prefix + "g")
            outs.append(self.n_heads)
        elif self.head_gate:
            raise ValueError("head gates beside biased projections are not built")
        self.qkv = Linear(names, hidden, outs, bias=self.has_bias, suffix="", bias_suffix=".b")
        self.o = Linear([prefix + "o"], self.n_heads * self.v_dim, [hidden], bias=self.has_bias, suffix="", bias_suffix=".b")
        self.q_norm_w = self.k_norm_w = self.conv_w = self.sink = None

    @property
    def W(self) -> int:
        """The projected row without the gate's logits."""
        return self.Wq + ((self.Wk + self.Wv) if self.own_kv else 0)

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.n_kv_heads, _page_row(self.head_dim), v_dim=_page_row(self.v_dim))

    def state_spec(self) -> Optional[StateSpec]:
        if self.conv_taps > 1:
            return StateSpec((self.conv_taps - 1, self.W), torch.float32)
        return None

    def tensor_specs(self) -> List[TensorSpec]:
        p = self.prefix
        specs = self.qkv.tensor_specs() + self.o.tensor_specs()
        if self.whole_norm:
            specs.append(TensorSpec(p + "q.norm", (self.Wq,), "norm"))
            if self.own_kv:
                specs.append(TensorSpec(p + "k.norm", (self.Wk,), "norm"))
        if self.learned_sink:
            specs.append(TensorSpec(p + "sink", (self.n_heads,), "sink"))
        if self.conv_taps:
            specs += [TensorSpec(p + n + ".conv", (w, self.conv_taps), "taps") for n, w in (("q", self.Wq), ("k", self.Wk), ("v", self.Wv))]
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.qkv.bind(get, rt)
        self.o.bind(get, rt)
        f32 = lambda name: get(self.prefix + name).to(device=rt.device, dtype=torch.float32).contiguous()
        if self.whole_norm:
            self.q_norm_w = f32("q.norm")
            self.k_norm_w = f32("k.norm") if self.own_kv else None
        if self.conv_taps:
            self.conv_w = torch.cat([f32("q.conv"), f32("k.conv"), f32("v.conv")], dim=0).contiguous()     # [W, taps]
            # one tap reads no row before the present one: the kernel is handed a state without rows
            self._no_state = torch.zeros((1, 0, self.W), dtype=torch.float32, device=rt.device)
        if self.unit_sink:
            self.sink = torch.zeros(self.n_heads, dtype=torch.float32, device=rt.device)     # a sink whose score is 0
        if self.learned_sink:
            self.sink = f32("sink")
        if self.position is not None and getattr(self.position, "inv_freq", None) is None:
            self.position.bind(get, rt)

    def forward(self, ctx: StepContext, h, cache: LayerCache, residual: Optional[Residual] = None):
        W, nq = self.W, self.Wq
        if not self.own_kv and cache.writes:
            raise RuntimeError("a layer without keys and values of its own reads another run's pages: the schedule must say whose")
        rows = self.qkv.product(h, f32_ok=True)
        gate = None
        if self.conv_taps or self.head_gate or rows.dtype != torch.float32:
            rows = K.sum_parts(rows, None, torch.float32)             # plain rows [T, W (+ heads)]
            if self.head_gate:
                gate = rows[:, W:W + self.n_heads]
        mark(ctx, "qkv")
        if self.conv_taps:
            # (a run that reads another's cache has no state of its own to convolve with: not built)
            if cache.state is None and self.conv_taps > 1:
                raise RuntimeError("a convolution behind the projections needs the run's own state")
            state = cache.state if self.conv_taps > 1 else self._no_state
            rows = K.causal_conv(ctx, rows[:, :W], self.conv_w, state, torch.float32, add_input=False)
            mark(ctx, "conv")
        cs, rot, pairing = None, 0, 0
        if self.position is not None:
            cs, rot, pairing = self.position.prepare(ctx), self.position.rot, self.position.pairing
        q = K.qkv_prepare(ctx, rows, self.qkv.bias, self.rt.dtype, self.n_heads, self.n_kv_heads, self.head_dim, self.v_dim,
                          self.q_norm_w, self.k_norm_w, self.eps, self.temp_coef, self.temp_every, cache.k_pool, cache.v_pool,
                          cache.table, writes=cache.writes, cs=cs, rot=rot, pairing=pairing)
        mark(ctx, "prepare")
        a = K.capped_attention(ctx, q, cache.k_pool, cache.v_pool, cache.table, self.n_heads, self.n_kv_heads, self.head_dim,
                               self.v_dim, self.scale, self.softcap, self.sink, gate)
        mark(ctx, "attention")
        out = self.o.add_to(a, residual) if residual is not None else None
        if out is None:
            out = self.o.product(a, f32_ok=True)
            if self.o.bias is not None:
                out = K.sum_parts(out, self.o.bias, torch.float32)
        mark(ctx, "o")
        return out
