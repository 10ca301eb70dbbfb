"""SwiGLU feed-forward: d = (silu(x Wg^T) * (x Wu^T)) Wd^T without biases
(reference: Daisi.Llogos/Inference/ForwardPass.cs:240-246; silu Daisi.Llogos.Cpu/Silu.cs:9-16).
Gate and up are one stacked product whose row is [gate | up]."""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

import torch

import math

from ..ops import kernels as K
from .base import FeedForward, Residual, Runtime, StepContext, TensorSpec, mark, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True
    takes_normed_rows = True
    adds_to_residual = True

    def __init__(self, prefix: str, hidden: int, intermediate: int,
                 names: Sequence[str] = ("gate_proj", "up_proj", "down_proj"), suffix: str = ".weight"):
        """names, suffix: the three matrices' tensor names behind `prefix`."""
        self.prefix = prefix
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear([prefix + names[0], prefix + names[1]], hidden, [intermediate, intermediate], gated=True, suffix=suffix)
        self.down = Linear([prefix + names[2]], intermediate, [hidden], suffix=suffix)

    def tensor_specs(self) -> List[TensorSpec]:
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.gate_up.bind(get, rt)
        self.down.bind(get, rt)

    def forward(self, ctx: StepContext, h, residual: Optional[Residual] = None):
        act = self.gate_up.gated_product(h)
        if act is not None:
            # on packed weights silu(gate) * up is the epilogue of the gate/up product
            # (the reference's MatMulSwiGLU, Daisi.Llogos/IComputeBackend.cs:448-456)
            mark(ctx, "gate_up")
            out = self.down.add_to(act, residual) if residual is not None else None
            if out is None:
                out = self.down.product(act, f32_ok=True)
            mark(ctx, "down")
            return out
        gu = self.gate_up.product(h)
        mark(ctx, "gate_up")
        # otherwise silu(gate) * up is made inside the down product where its kernel can (few rows), by a
        # kernel of its own for many; the residual sum that follows adds the product's parts
        out = self.down.product(gu, swiglu_input=True, f32_ok=True)
        mark(ctx, "down")
        return out


def _softplus(z: float) -> float:
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


@register_feed_forward("activated")
class ActivatedMLP(FeedForward):
    """d = W_down act(W_up h) with an activation from ops.kernels.ACTIVATIONS.  'xielu' has two learned
    numbers (p, q) in the tensor `prefix + "act"`: z > 0: softplus(p) z^2 + z / 2; z <= 0:
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2; the two softplus values are worked out once, when
    the tensor is bound."""
    graph_safe = True

    def __init__(self, prefix: str, hidden: int, intermediate: int, activation: str = "xielu", suffix: str = ""):
        if activation not in K.ACTIVATIONS:
            raise ValueError(f"unknown activation '{activation}'; known: {sorted(K.ACTIVATIONS)}")
        self.prefix, self.hidden, self.intermediate, self.activation = prefix, int(hidden), int(intermediate), activation
        self.up = Linear([prefix + "up"], hidden, [intermediate], suffix=suffix)
        self.down = Linear([prefix + "down"], intermediate, [hidden], suffix=suffix)
        self.a = self.b = 0.0

    def tensor_specs(self) -> List[TensorSpec]:
        specs = self.up.tensor_specs() + self.down.tensor_specs()
        if self.activation == "xielu":
            specs.append(TensorSpec(self.prefix + "act", (2,), "shape"))
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        self.up.bind(get, rt)
        self.down.bind(get, rt)
        if self.activation == "xielu":
            p, q = (float(v) for v in get(self.prefix + "act").to(torch.float32).reshape(-1).tolist())
            self.a, self.b = _softplus(p), 0.5 + _softplus(q)

    def forward(self, ctx: StepContext, h):
        z = self.up.product(h, f32_ok=True)
        mark(ctx, "up")
        act = K.activation(z, self.activation, self.rt.dtype, self.a, self.b)
        out = self.down.product(act, f32_ok=True)
        mark(ctx, "down")
        return out
