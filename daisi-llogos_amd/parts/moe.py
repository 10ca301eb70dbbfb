"""A mixture of experts without a router: a table over token ids names each token's experts.

    out_t = (1 / top) sum_j expert_(table[id_t, j])(h_t)  +  sigmoid(w_sg . h_t) * shared(h_t)
    expert(h) = W_down act(W_up h)          (no biases; the shared expert has the same form)

The table is an integer tensor [vocab, top] whose rows hold different experts.  The choice is made
on the device from the step's ids, so single-token steps can be captured and replayed.  The
experts' matrices are stacked ([experts, ff, width] and [experts, width, ff]); the (token, choice)
pairs are sorted by expert and each expert's rows multiplied tile by tile."""
from __future__ import annotations

import os
from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import FeedForward, Runtime, StepContext, TensorSpec, mark, register_feed_forward
from .linear import Linear

_EPILOGUES = ("relu2",)        # activations that the experts' product applies in its epilogue


def _float32(product: torch.Tensor) -> torch.Tensor:
    """A product as float32 (in parts or not), for consumers that read nothing else."""
    return product if product.dtype == torch.float32 else K.sum_parts(product, None, torch.float32)


@register_feed_forward("table_moe")
class TableMoE(FeedForward):
    graph_safe = True

    def __init__(self, prefix: str, hidden: int, vocab: int, n_experts: int, top: int, intermediate: int,
                 shared_intermediate: int = 0, activation: str = "relu2"):
        if not 1 <= top <= n_experts <= K.MOE_MAX_EXPERTS:
            raise ValueError(f"top {top} of {n_experts} experts: outside 1..experts..{K.MOE_MAX_EXPERTS}")
        if activation not in _EPILOGUES:
            raise ValueError(f"unknown expert activation '{activation}'; known: {list(_EPILOGUES)}")
        self.prefix, self.hidden, self.vocab = prefix, int(hidden), int(vocab)
        self.n_experts, self.top, self.intermediate = int(n_experts), int(top), int(intermediate)
        self.shared_intermediate, self.activation = int(shared_intermediate), activation
        self.table = self.up = self.down = None
        self.shared_up = self.shared_down = None
        if self.shared_intermediate:
            # the gate's row rides behind the shared expert's up matrix: one product for both
            self.shared_up = Linear([prefix + "shared.up", prefix + "shared.sg"], hidden, [self.shared_intermediate, 1], suffix="")
            self.shared_down = Linear([prefix + "shared.down"], self.shared_intermediate, [hidden], suffix="")

    def tensor_specs(self) -> List[TensorSpec]:
        p = self.prefix
        specs = []
        for e in range(self.n_experts):
            specs += [TensorSpec(f"{p}e{e}.up", (self.intermediate, self.hidden), "matrix"),
                      TensorSpec(f"{p}e{e}.down", (self.hidden, self.intermediate), "matrix")]
        specs.append(TensorSpec(p + "table", (self.vocab, self.top), f"choices:{self.n_experts}"))
        if self.shared_up is not None:
            specs += self.shared_up.tensor_specs() + self.shared_down.tensor_specs()
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        p, E = self.prefix, self.n_experts
        self.up = torch.empty((E, self.intermediate, self.hidden), dtype=rt.dtype, device=rt.device)
        self.down = torch.empty((E, self.hidden, self.intermediate), dtype=rt.dtype, device=rt.device)
        for e in range(E):
            self.up[e].copy_(get(f"{p}e{e}.up"))
            self.down[e].copy_(get(f"{p}e{e}.down"))
        table = get(p + "table")
        if table.dtype.is_floating_point:
            raise ValueError(f"{p}table must hold integers")
        table = table.to(torch.int64)
        if table.numel() and (int(table.min()) < 0 or int(table.max()) >= E):
            raise ValueError(f"{p}table names experts outside 0..{E - 1}")
        self.table = table.to(device=rt.device, dtype=torch.int32).contiguous()
        if self.shared_up is not None:
            self.shared_up.bind(get, rt)
            self.shared_down.bind(get, rt)

    def matrix_elements(self) -> int:
        """What a token is multiplied with: its `top` experts and the shared one."""
        return super().matrix_elements() + 2 * self.top * self.intermediate * self.hidden

    def forward(self, ctx: StepContext, h: torch.Tensor):
        order, seg, where = K.moe_route(ctx.ids, self.table, self.n_experts)
        act = K.moe_product(h, self.up, order, seg, self.top, True, self.rt.dtype, relu2=True)
        y = K.moe_product(act, self.down, order, seg, self.top, False, torch.float32)
        mark(ctx, "experts")
        shared = gate = None
        if self.shared_up is not None:
            z = _float32(self.shared_up.product(h, f32_ok=True))             # [(parts,) T, ff + 1]
            a = K.activation(z, self.activation, self.rt.dtype, cols=self.shared_intermediate)
            shared = _float32(self.shared_down.product(a, f32_ok=True))
            gate = z[..., self.shared_intermediate:]
            mark(ctx, "shared")
        out = K.moe_combine(y, where, self.top, shared, gate)
        mark(ctx, "combine")
        return out


@register_feed_forward("routed_moe")
class RoutedMoE(FeedForward):
    """A mixture of gated experts chosen by a router, beside an optional shared expert:

        z = W_router h (32-bit);  s = softmax(z) over all router outputs
        choice scores c = s + correction; the outputs form `groups` equal groups of neighbours, a group's score is
        its largest c, and only outputs of the `keep` best groups can be chosen; the `top` largest c are chosen
        weights w_j = s_j / (sum of the chosen s + 1e-20) * scale
        out = sum_j w_j expert_j(h)  +  shared(h),     expert(h) = W_down (silu(W_gate h) * (W_up h))

    The last `identity` router outputs have no matrices: such an expert returns h itself.  The choice, the
    sorting of the (token, choice) pairs by expert and the weighted sum are made on the device, so single-token
    steps are captured and replayed.  An expert's gate and up matrices are stacked with their rows in turn
    (gate 0, up 0, gate 1, ...), so that a gate's and an up's sum of one column meet in one thread of the
    experts' product, which writes silu(gate) * up alone.

    The shared expert depends on h alone, so in steps of few rows, whose kernels are short and wait for one another,
    it is queued on a second stream beside the router and the chosen experts (inside a captured step the two become
    branches of the graph); both streams meet before the weighted sum.  Every use of the second stream begins by
    waiting for the first, so memory that either stream's allocator hands out again is no longer read by the other.
    It pays where the shared expert's matrices are large (8 layers at batch 8 and 1: 4,096 wide with 176 MB of them
    2,429 -> 2,335 us and 1,529 -> 1,470 us a step; 2,048 wide with 50 MB 1,457 -> 1,469 and 1,012 -> 1,037), so it is
    taken from `side_bytes` of shared matrices on.  `LLOGOS_PARALLEL_STREAMS=0` keeps everything on one stream."""
    graph_safe = True
    side_rows = 0 if os.environ.get("LLOGOS_PARALLEL_STREAMS", "1") == "0" else 64     # steps of up to so many rows use the second stream
    side_bytes = 64 << 20        # ... when the shared expert's matrices take at least so many bytes
    _side_streams = {}

    def __init__(self, prefix: str, hidden: int, n_experts: int, top: int, intermediate: int, identity: int = 0,
                 groups: int = 1, keep: int = 1, scale: float = 1.0, shared_intermediate: int = 0, correction: bool = True):
        total = int(n_experts) + int(identity)
        if not 1 <= top <= total <= K.MOE_MAX_EXPERTS:
            raise ValueError(f"top {top} of {total} router outputs: outside 1..outputs..{K.MOE_MAX_EXPERTS}")
        if groups < 1 or total % groups or not 1 <= keep <= groups or keep * (total // groups) < top:
            raise ValueError(f"{groups} groups of which {keep} are kept do not fit {total} router outputs and top {top}")
        self.prefix, self.hidden = prefix, int(hidden)
        self.n_experts, self.identity, self.top, self.intermediate = int(n_experts), int(identity), int(top), int(intermediate)
        self.groups, self.keep, self.scale = int(groups), int(keep), float(scale)
        self.shared_intermediate, self.has_correction = int(shared_intermediate), bool(correction)
        self.router_w = self.correction = self.gate_up = self.down = None
        self.shared = None
        self.probed = None          # {"choice": int32 [T, top]} of the last step that was run part by part (measurements)
        if self.shared_intermediate:
            from .mlp import SwiGLU
            self.shared = SwiGLU(prefix + "shared.", hidden, self.shared_intermediate, names=("gate", "up", "down"), suffix="")

    @property
    def outputs(self) -> int:
        return self.n_experts + self.identity

    def tensor_specs(self) -> List[TensorSpec]:
        p = self.prefix
        specs = []
        for e in range(self.n_experts):
            specs += [TensorSpec(f"{p}e{e}.gate", (self.intermediate, self.hidden), "matrix"),
                      TensorSpec(f"{p}e{e}.up", (self.intermediate, self.hidden), "matrix"),
                      TensorSpec(f"{p}e{e}.down", (self.hidden, self.intermediate), "matrix")]
        specs.append(TensorSpec(p + "router", (self.outputs, self.hidden), "router"))
        if self.has_correction:
            specs.append(TensorSpec(p + "correction", (self.outputs,), "correction"))
        if self.shared is not None:
            specs += self.shared.tensor_specs()
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        p, E, F = self.prefix, self.n_experts, self.intermediate
        if E:
            self.gate_up = torch.empty((E, 2 * F, self.hidden), dtype=rt.dtype, device=rt.device)
            self.down = torch.empty((E, self.hidden, F), dtype=rt.dtype, device=rt.device)
            for e in range(E):
                self.gate_up[e, 0::2].copy_(get(f"{p}e{e}.gate"))
                self.gate_up[e, 1::2].copy_(get(f"{p}e{e}.up"))
                self.down[e].copy_(get(f"{p}e{e}.down"))
        self.router_w = get(p + "router").to(device=rt.device, dtype=torch.float32).contiguous()
        self.correction = get(p + "correction").to(device=rt.device, dtype=torch.float32).contiguous() if self.has_correction else None
        if self.shared is not None:
            self.shared.bind(get, rt)

    def matrix_elements(self) -> int:
        """What a token is multiplied with: the router, its `top` experts (as if all had matrices) and the shared one."""
        return super().matrix_elements() + self.outputs * self.hidden + 3 * self.top * self.intermediate * self.hidden

    def forward(self, ctx: StepContext, h: torch.Tensor):
        shared, side = None, None
        if self.shared is not None and h.shape[0] <= self.side_rows and (ctx is None or ctx.probe is None) and h.is_cuda \
                and 3 * self.shared_intermediate * self.hidden * h.element_size() >= self.side_bytes:
            main = torch.cuda.current_stream(h.device)
            side = self._side_streams.get(h.device)
            if side is None:
                side = self._side_streams[h.device] = torch.cuda.Stream(device=h.device)
            side.wait_stream(main)                       # h is there
            with torch.cuda.stream(side):
                shared = _float32(self.shared.forward(ctx, h))
        choice, weight = K.moe_router(h, self.router_w, self.correction, self.groups, self.keep, self.top, self.scale)
        mark(ctx, "router")
        if ctx is not None and ctx.probe is not None:
            self.probed = {"choice": choice}
        T, W = h.shape
        if self.n_experts:
            order, seg, where = K.moe_route(None, choice, self.outputs)
            act = K.moe_product(h, self.gate_up, order, seg, self.top, True, self.rt.dtype, gated=True)
            y = K.moe_product(act, self.down, order, seg, self.top, False, torch.float32)
        else:
            where = torch.zeros(T * self.top, dtype=torch.int32, device=h.device)
            y = torch.zeros((T * self.top, W), dtype=torch.float32, device=h.device)
        mark(ctx, "experts")
        if side is not None:
            torch.cuda.current_stream(h.device).wait_stream(side)
        elif self.shared is not None:
            shared = _float32(self.shared.forward(ctx, h))
            mark(ctx, "shared")
        out = K.moe_combine_weighted(y, where, choice, weight, self.n_experts, h, shared)
        mark(ctx, "combine")
        return out
