"""A recurrent mixer with a real-gated linear recurrent unit: two branches of `width` channels,

    y = gelu_tanh(W_y h + b_y)                                   the gate branch
    u = conv(W_x h + b_x) + b_c                                  a short causal convolution over time, a channel at a time
    r = sigmoid(R_b u_b + b_r),  i = sigmoid(I_b u_b + b_i)      block by block: the channels are cut into `blocks` equal
                                                                 parts, each with square matrices of its own
    a = exp(-sharpness * r * softplus(lam))
    S <- a S + sqrt(1 - a^2) * (i * u)                           one number a channel and sequence, from S = 0
    out = W_o (S * y)

The two branches are one stacked product, and so are the two gates of a block.  A sequence's state is the
convolution's last taps - 1 inputs and S, rows of one per-slot tensor [taps, width] (float32).  Everything behind the
projections is 32-bit: convolution, gate logits, sigmoids, decay, recurrence."""
from __future__ import annotations

import math
from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Runtime, StateSpec, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear


@register_mixer("rglru")
class RGLRU(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden: int, width: int, blocks: int, conv_taps: int, sharpness: float = 8.0):
        if width <= 0 or blocks <= 0 or width % blocks:
            raise ValueError(f"{width} channels do not divide into {blocks} blocks")
        if not 1 <= conv_taps <= K.MAX_CONV_TAPS:
            raise ValueError(f"a convolution of {conv_taps} taps is outside 1..{K.MAX_CONV_TAPS}")
        self.prefix, self.hidden, self.width, self.blocks, self.taps = prefix, int(hidden), int(width), int(blocks), int(conv_taps)
        self.block = self.width // self.blocks
        self.sharpness = float(sharpness)
        self.yx = Linear([prefix + "y", prefix + "x"], hidden, [self.width, self.width], bias=True, suffix="", bias_suffix=".b")
        self.o = Linear([prefix + "o"], self.width, [hidden], suffix="")
        self.conv_w = self.conv_b = self.gate_w = self.r_bias = self.i_bias = self.decay = None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.taps, self.width), torch.float32)        # taps - 1 rows of inputs, then S

    def kv_spec(self) -> Optional[KVSpec]:
        return None

    def tensor_specs(self) -> List[TensorSpec]:
        p, C, nb, bs = self.prefix, self.width, self.blocks, self.block
        return self.yx.tensor_specs() + [
            TensorSpec(p + "conv", (C, self.taps), "taps"), TensorSpec(p + "conv.b", (C,), "bias"),
            TensorSpec(p + "ra", (nb, bs, bs), "matrix"), TensorSpec(p + "ra.b", (nb, bs), "bias"),
            TensorSpec(p + "ri", (nb, bs, bs), "matrix"), TensorSpec(p + "ri.b", (nb, bs), "bias"),
            TensorSpec(p + "lam", (C,), "bonus")] + self.o.tensor_specs()

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.yx.bind(get, rt)
        self.o.bind(get, rt)
        f32 = lambda name: get(self.prefix + name).to(device=rt.device, dtype=torch.float32).contiguous()
        self.conv_w, self.conv_b = f32("conv"), f32("conv.b")
        # a block's two gate matrices one above the other: [blocks, 2 * block, block]; their values are the
        # checkpoint's (bfloat16 numbers are float32 numbers), and the logits are summed in 32-bit
        ra = get(self.prefix + "ra").to(device=rt.device, dtype=rt.dtype)
        ri = get(self.prefix + "ri").to(device=rt.device, dtype=rt.dtype)
        self.gate_w = torch.cat([ra, ri], dim=1).contiguous()
        self.gate_w_kn = self.gate_w.transpose(1, 2).contiguous()      # k-major, for steps of few rows
        self.r_bias, self.i_bias = f32("ra.b").reshape(-1).contiguous(), f32("ri.b").reshape(-1).contiguous()
        # sharpness * softplus(lam), once, in float32
        self.decay = (torch.nn.functional.softplus(f32("lam")) * self.sharpness).contiguous()

    def matrix_elements(self) -> int:
        return self.yx.matrix_elements() + self.o.matrix_elements() + 2 * self.width * self.block

    def forward(self, ctx: StepContext, h, cache: LayerCache):
        C, T = self.width, ctx.n_tokens
        if cache.state is None:
            raise RuntimeError("the recurrent mixer needs its per-sequence state")
        rows = K.sum_parts(self.yx.product(h, f32_ok=True), self.yx.bias, torch.float32)       # [T, 2 C]: y logits | conv input
        mark(ctx, "yx")
        u = K.causal_conv(ctx, rows[:, C:], self.conv_w, cache.state, torch.float32, add_input=False, bias=self.conv_b)
        mark(ctx, "conv")
        gates = torch.empty((T, self.blocks, 2 * self.block), dtype=torch.float32, device=u.device)
        K.head_products(u.view(T, self.blocks, self.block), self.gate_w, gates, self.gate_w_kn)
        mark(ctx, "gates")
        s = K.gated_recurrence(ctx, u, gates.view(T, 2 * C), self.block, self.r_bias, self.i_bias, self.decay, rows[:, :C],
                               cache.state[:, self.taps - 1, :], self.rt.dtype)
        mark(ctx, "recurrence")
        out = self.o.product(s, f32_ok=True)
        mark(ctx, "o")
        return out
