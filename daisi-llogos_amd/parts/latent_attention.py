"""Attention through a low-rank latent, with an optional learned sink in the softmax and an optional
sigmoid gate on every head's output.

    c_q = norm(W_dq h);  q = W_uq c_q                    per head [dim unrotated | rot rotated]
                                                         (q_rank 0: q = W_q h, no latent on the query's side)
    [c_raw | k_rot] = W_dkv h;  c = norm(c_raw)          the latent, and one rotated key part for all heads
    k_h = W_uk,h c;  v_h = W_uv,h c
    score_h(i, j) = (q_h,plain(i) . k_h(j) + q_h,rot(i) . k_rot(j)) * scale,   j <= i
    weights = exp(score) / (sum_j exp(score) [+ exp(sink_h)])
    out = W_o [sigmoid(W_g h)_h * sum_j weights_h(i, j) v_h(j)]_h            (the gate is optional)

The cache holds one row [c | k_rot] a token, which serves every head, and no values of its own.
The scores are taken in the latent's space, q_h,plain . W_uk,h c = (W_uk,h^T q_h,plain) . c, so a
head's query becomes [W_uk,h^T q_h,plain | q_h,rot] against the cached row, the weighted sum runs
over latents, and W_uv,h is applied to that sum (the gate in that product's epilogue).  The
projections that read h (q or dq, dkv, g) are one stacked product.

Whole prompts in bfloat16 whose head shapes the matrix cores' attention takes, and that have no rotated
part, go the other way round: the step's latents are multiplied with all heads' key and value matrices at
once (one product of the library's kind), the keys and values go to pages of the step's own, and the
prompt kernel of the attention with keys and values a head runs on them: a quarter or less of the
arithmetic of scores and sums over latents, on the faster kernel.  The cache still gets the latents alone."""
from __future__ import annotations

from typing import Callable, List, Optional

import torch

from ..ops import kernels as K
from .base import KVSpec, LayerCache, Mixer, Runtime, StepContext, TensorSpec, mark, register_mixer
from .linear import Linear
from .rope import Rotary


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, hidden: int, n_heads: int, dim: int, rot_dim: int, v_dim: int, q_rank: int,
                 kv_rank: int, scale: float, eps: float, position: Optional[Rotary] = None, sink: bool = True,
                 suffix: str = "", head_gate: bool = False):
        self.prefix, self.hidden = prefix, int(hidden)
        self.n_heads, self.dim, self.rot_dim, self.v_dim = int(n_heads), int(dim), int(rot_dim), int(v_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.position = position
        self.has_sink, self.head_gate = bool(sink), bool(head_gate)
        if position is not None and (position.pairing != 1 or position.rot > self.rot_dim):
            raise ValueError("the rotated key part takes neighbouring pairs, at most rot_dim dimensions")
        # the cached row [latent | rotated part], widened to the pages' step of 16 dimensions
        self.row = -(-(self.kv_rank + self.rot_dim) // K.HEAD_DIM_STEP) * K.HEAD_DIM_STEP
        if self.row > 1024:
            raise ValueError(f"a cached row of {self.row} values is more than the attention kernel takes (1024)")
        H = self.n_heads
        # what reads h beside the query's latent, stacked: [q (without a latent of its own) | dkv | g]
        self.q_width = 0 if self.q_rank else H * (self.dim + self.rot_dim)
        names, outs = [prefix + "dkv"], [self.kv_rank + self.rot_dim]
        if not self.q_rank:
            names, outs = [prefix + "q"] + names, [self.q_width] + outs
        if self.head_gate:
            names.append(prefix + "g")
            outs.append(H)
        self.inp = Linear(names, hidden, outs, suffix=suffix)
        self.dq = Linear([prefix + "dq"], hidden, [self.q_rank], suffix=suffix) if self.q_rank else None
        self.uq = Linear([prefix + "uq"], self.q_rank, [H * (self.dim + self.rot_dim)], suffix=suffix) if self.q_rank else None
        self.o = Linear([prefix + "o"], H * self.v_dim, [hidden], suffix=suffix)
        self.uk_t = self.uv = self.uk_kn = self.uv_kn = self.q_norm_w = self.c_norm_w = self.sink = None
        self.ukv = None              # [uk ; uv] stacked by rows, for whole prompts
        self.prompt_rows = 128       # steps of at least so many tokens that are all whole prompts make keys and values a head

    def _linears(self) -> List[Linear]:
        return [lin for lin in (self.dq, self.uq, self.inp, self.o) if lin is not None]

    @property
    def head_dim(self) -> int:         # (what Model.step_flops takes as the width of a head's dot products)
        return self.row

    def kv_spec(self) -> KVSpec:
        # the matrix cores' attention (bfloat16, rows up to its limit) reads values in an operand order of their
        # own: the latent is then cached a second time, as a value row; otherwise a value is part of its key row
        rt = getattr(self, "rt", None)
        mfma = rt is not None and rt.dtype == torch.bfloat16 and self.row <= K.LATENT_MFMA_MAX_ROW
        return KVSpec(1, self.row, values=mfma)

    def tensor_specs(self) -> List[TensorSpec]:
        p, H = self.prefix, self.n_heads
        specs = [s for lin in self._linears() for s in lin.tensor_specs()]
        if self.q_rank:
            specs.append(TensorSpec(p + "dq.norm", (self.q_rank,), "norm"))
        specs += [TensorSpec(p + "dkv.norm", (self.kv_rank,), "norm"),
                  TensorSpec(p + "uk", (H * self.dim, self.kv_rank), "matrix"),
                  TensorSpec(p + "uv", (H * self.v_dim, self.kv_rank), "matrix")]
        if self.has_sink:
            specs.append(TensorSpec(p + "sink", (H,), "sink"))
        return specs

    def bind(self, get: Callable[[str], Optional[torch.Tensor]], rt: Runtime) -> None:
        super().bind(get, rt)
        for lin in self._linears():
            lin.bind(get, rt)
        H = self.n_heads
        f32 = lambda name: get(self.prefix + name).to(device=rt.device, dtype=torch.float32).contiguous()
        self.q_norm_w, self.c_norm_w = (f32("dq.norm") if self.q_rank else None), f32("dkv.norm")
        self.sink = f32("sink") if self.has_sink else None
        uk = get(self.prefix + "uk").to(device=rt.device, dtype=rt.dtype)
        # per head the transposed key matrix [rank, dim]: a query's unrotated part times it is the query in the latent's space
        self.uk_t = uk.view(H, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.uv = get(self.prefix + "uv").to(device=rt.device, dtype=rt.dtype).view(H, self.v_dim, self.kv_rank).contiguous()
        # the same two sets of matrices k-major, for steps of few rows (a few MB a layer)
        self.uk_kn = uk.view(H, self.dim, self.kv_rank).contiguous()
        self.uv_kn = self.uv.transpose(1, 2).contiguous()
        if self._heads_on_matrix_cores():
            self.ukv = torch.cat([uk, self.uv.view(H * self.v_dim, self.kv_rank)], dim=0).contiguous()
        if self.position is not None and getattr(self.position, "inv_freq", None) is None:
            self.position.bind(get, rt)

    def matrix_elements(self) -> int:
        return super().matrix_elements() + self.n_heads * self.kv_rank * (self.dim + self.v_dim)

    def _heads_on_matrix_cores(self) -> bool:
        """Whether whole prompts can run as attention with keys and values a head (see the module's text)."""
        return self.rt.dtype == torch.bfloat16 and self.rot_dim == 0 and not self.q_rank and self.dim in (64, 96, 128) \
            and self.v_dim in (64, 80, 96, 128)

    @staticmethod
    def _prompt_pages(ctx: StepContext):
        """Pages of the step's own for whole prompts: (number of pages, table int32 [batch, pages of the longest]), sequence
        after sequence; made once a step on the device from the step's token offsets."""
        made = ctx.shared.get("prompt_pages")
        if made is None:
            lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
            pages = [-(-n // K.PAGE_TOKENS) for n in lens]
            counts = (ctx.cu_dev[1:] - ctx.cu_dev[:-1] + (K.PAGE_TOKENS - 1)) // K.PAGE_TOKENS
            first = torch.cumsum(counts, 0) - counts
            table = (first[:, None] + torch.arange(max(pages), device=first.device)[None, :]).to(torch.int32).contiguous()
            made = ctx.shared["prompt_pages"] = (sum(pages), table)
        return made

    def _forward_prompt(self, ctx: StepContext, rows: torch.Tensor, kv: torch.Tensor, gate, cache: LayerCache) -> torch.Tensor:
        f32, H, T = torch.float32, self.n_heads, ctx.n_tokens
        qa = torch.empty((T, H, self.row), dtype=self.rt.dtype, device=rows.device)       # (no rotated part: nothing is written)
        c = torch.empty((T, self.kv_rank), dtype=self.rt.dtype, device=rows.device)
        K.latent_prepare(ctx, kv, rows[:, :self.q_width], qa, self.c_norm_w, self.eps, None, cache.k_pool, cache.v_pool, cache.table,
                         H, self.dim, 0, 0, self.kv_rank, c_out=c)
        keys_values = K.sum_parts(K.gemm_product(c, self.ukv, self.rt.dtype, f32_ok=True), None, f32)     # [T, H * (dim + v_dim)]
        mark(ctx, "rotation")
        n_pages, table = self._prompt_pages(ctx)
        k_pool = torch.empty((n_pages, H, K.PAGE_TOKENS * self.dim), dtype=self.rt.dtype, device=rows.device)
        v_pool = torch.empty((n_pages, H, K.PAGE_TOKENS * self.v_dim), dtype=self.rt.dtype, device=rows.device)
        q = K.qkv_prepare(ctx, rows, None, self.rt.dtype, H, H, self.dim, self.v_dim, None, None, self.eps, 0.0, 1, k_pool, v_pool,
                          table, kv_rows=keys_values)
        a = K.capped_attention(ctx, q, k_pool, v_pool, table, H, H, self.dim, self.v_dim, self.scale, 0.0, self.sink, gate)
        mark(ctx, "attention")
        out = self.o.product(a, f32_ok=True)
        mark(ctx, "o")
        return out

    def forward(self, ctx: StepContext, h: torch.Tensor, cache: LayerCache) -> torch.Tensor:
        f32, H, T = torch.float32, self.n_heads, ctx.n_tokens
        plain = lambda p: K.sum_parts(p, None, f32)          # (a product may come as partial sums of a split along k)
        rows = plain(self.inp.product(h, f32_ok=True))                            # [T, (q) | rank + rot | (heads)]
        kv = rows[:, self.q_width:self.q_width + self.kv_rank + self.rot_dim]
        gate = rows[:, self.q_width + self.kv_rank + self.rot_dim:] if self.head_gate else None
        if self.q_rank:
            cq = plain(self.dq.product(h, f32_ok=True))
            cq = K.rmsnorm(cq, self.q_norm_w, self.eps, self.rt.dtype)
            q = plain(self.uq.product(cq, f32_ok=True))                           # [T, H * (dim + rot)]
        else:
            q = rows[:, :self.q_width]
        mark(ctx, "projections")
        if self.ukv is not None and not ctx.is_decode and not ctx.in_graph and T >= self.prompt_rows and ctx.cu_dev is not None \
                and not any(ctx.starts):
            return self._forward_prompt(ctx, rows, kv, gate, cache)
        cs = self.position.prepare(ctx) if self.position is not None else None
        qa = torch.empty((T, H, self.row), dtype=self.rt.dtype, device=h.device)
        K.latent_prepare(ctx, kv, q, qa, self.c_norm_w, self.eps, cs, cache.k_pool, cache.v_pool, cache.table, H, self.dim, self.rot_dim,
                         self.position.rot if self.position is not None else 0, self.kv_rank)
        K.head_products(q.unflatten(1, (H, self.dim + self.rot_dim))[:, :, :self.dim], self.uk_t, qa[:, :, :self.kv_rank], self.uk_kn)
        mark(ctx, "rotation")
        lat = None
        if cache.v_pool is not None:
            lat = K.latent_attention_mfma(ctx, qa, cache.k_pool, cache.v_pool, cache.table, H, self.row, self.kv_rank, self.scale, self.sink)
        if lat is None:
            lat = K.attention_generic(qa, H * self.row, cache.k_pool, None, cache.table, ctx.tok_seq, ctx.tok_pos, H, 1, self.row,
                                      self.scale, v_dim=self.kv_rank, head_sink=self.sink)
        mark(ctx, "attention")
        a = torch.empty((T, H, self.v_dim), dtype=self.rt.dtype, device=h.device)
        K.head_products(lat.view(T, H, self.kv_rank), self.uv, a, self.uv_kn, gate=gate)
        out = self.o.product(a.view(T, H * self.v_dim), f32_ok=True)
        mark(ctx, "o")
        return out
