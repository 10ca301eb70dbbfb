"""Arrangement of a layer's parts.  The pre-norm residual block:

    x += pending;  a = mixer(norm1(x));  x += a;  d = ffn(norm2(x));  pending = d

Each residual sum is done inside the following norm's kernel, in float32, so the
feed-forward's output is handed on as `pending` and added by whoever norms next
(reference: the deferred adds of Daisi.Llogos/Inference/ForwardPass.cs:214-252); or, for
steps of few rows, by the product that closes the mixer or the feed-forward, which then also
leaves the following norm's rows for the product that opens the next part."""
from __future__ import annotations

import os
from typing import Callable, List, Optional, Tuple

import torch

from .base import Block, FeedForward, LayerCache, Mixer, Norm, NormedAhead, Part, Residual, Runtime, StepContext, TensorSpec, mark, register_block
from .norm import RMSNorm


@register_block("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn]

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    takes_next_norm = True

    def entry_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    @staticmethod
    def _norm(norm: Norm, x: torch.Tensor, delta, lazy: bool):
        # (only a norm that knows of unscaled rows is asked for them)
        return norm.forward(x, delta, lazy=True) if lazy and norm.takes_row_squares else norm.forward(x, delta)

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches, next_norm: Optional[Norm] = None):
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        # A part that says so may add its output to x itself and leave the next norm's rows half made
        # (then `a` or `d` is what it left, and the norm that takes it needs no kernel of its own).
        h = self._norm(self.mixer_norm, x, pending, self.mixer.takes_normed_rows)
        mark(ctx, "norm")
        if self.mixer.adds_to_residual and self.ffn_norm.takes_row_squares:
            a = self.mixer.forward(ctx, h, cache, residual=Residual(x, self.ffn_norm))
        else:
            a = self.mixer.forward(ctx, h, cache)
        mark(ctx, "mixer")
        h = self._norm(self.ffn_norm, x, a, self.ffn.takes_normed_rows)
        mark(ctx, "norm")
        if self.ffn.adds_to_residual and next_norm is not None and next_norm.takes_row_squares:
            d = self.ffn.forward(ctx, h, residual=Residual(x, next_norm))
        else:
            d = self.ffn.forward(ctx, h)
        mark(ctx, "feed_forward")
        return x, d


@register_block("sandwich")
class SandwichBlock(Block):
    """Norms before and after each sublayer, and optionally a short convolution over time on what a
    sublayer reads:

        x += post_mixer_norm(mixer(conv1(mixer_norm(x))));   x += post_ffn_norm(ffn(conv2(ffn_norm(x))))

    The feed-forward (with its norms and convolution) may be absent.  The normed outputs are float32
    deltas: the first is added by the kernel of the norm that follows, the second is handed on as
    `pending`.  The convolutions keep state for each sequence, so they are cache parts of the block
    beside its mixer."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, post_mixer_norm: Norm, ffn_norm: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None, post_ffn_norm: Optional[Norm] = None,
                 mixer_conv: Optional[Part] = None, ffn_conv: Optional[Part] = None):
        if (ffn is None) != (ffn_norm is None) or (ffn is None) != (post_ffn_norm is None):
            raise ValueError("a feed-forward comes with a norm before and a norm after it, or not at all")
        if ffn is None and ffn_conv is not None:
            raise ValueError("a convolution in front of a feed-forward that is not there")
        self.mixer_norm, self.mixer, self.post_mixer_norm = mixer_norm, mixer, post_mixer_norm
        self.ffn_norm, self.ffn, self.post_ffn_norm = ffn_norm, ffn, post_ffn_norm
        self.mixer_conv, self.ffn_conv = mixer_conv, ffn_conv

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn] if self.ffn is not None else []

    def cache_parts(self) -> List[Part]:
        return [p for p in (self.mixer_conv, self.mixer, self.ffn_conv) if p is not None]

    def parts(self) -> List[Part]:
        return [p for p in (self.mixer_norm, self.mixer_conv, self.mixer, self.post_mixer_norm, self.ffn_norm, self.ffn_conv,
                            self.ffn, self.post_ffn_norm) if p is not None]

    def entry_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    takes_next_norm = True

    def _read(self, ctx, norm: Norm, conv, x, delta, cache, want_f32: bool):
        """What a sublayer reads: norm(x + delta), through the convolution when there is one."""
        dtype = torch.float32 if want_f32 else self.rt.dtype
        if conv is None:
            return norm.forward(x, delta, out_dtype=dtype)
        h = norm.forward(x, delta, out_dtype=torch.float32)
        mark(ctx, "norm")
        return conv.forward(ctx, h, cache, out_dtype=dtype)

    def _close(self, x, out, post: Norm, nxt: Optional[Norm], rows_f32: bool):
        """A sublayer's output `out` joins the stream through its norm `post`, and the norm `nxt` that
        reads the stream next is applied on the way: one kernel for both where both are RMS norms over the
        stream's width (then x is complete and the rows are returned), else the norm's own kernel (then the
        normed output is returned as a delta that the next norm adds).  Returns (rows or None, delta or None).
        The rows handed to another block are float32 (a convolution or a mixer that mixes rows reads them)."""
        from ..ops import kernels as K
        fused = isinstance(post, RMSNorm) and (nxt is None or isinstance(nxt, RMSNorm)) and x.shape[1] * 4 <= 65536 \
            and (nxt is None or nxt.eps == post.eps)
        if not fused:
            a = out if (out.dim() == 2 and out.dtype == torch.float32) else K.sum_parts(out, None, torch.float32)
            return None, post.forward(a, out_dtype=torch.float32)
        dtype = torch.float32 if rows_f32 else self.rt.dtype
        rows = K.sandwich_norm(x, out, post.weight, nxt.weight if nxt is not None else None, post.eps, dtype)
        return rows, None

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches, next_norm: Optional[Norm] = None):
        caches = list(caches)
        conv1_cache = caches.pop(0) if self.mixer_conv is not None else None
        mixer_cache = caches.pop(0)
        conv2_cache = caches.pop(0) if self.ffn_conv is not None else None
        f32_in = self.mixer.takes_float32_rows
        h = self._read(ctx, self.mixer_norm, self.mixer_conv, x, pending, conv1_cache, f32_in)
        mark(ctx, "conv" if self.mixer_conv is not None else "norm")
        a = self.mixer.forward(ctx, h, mixer_cache)
        mark(ctx, "mixer")
        if self.ffn is None:
            rows, delta = self._close(x, a, self.post_mixer_norm, next_norm, True)
            mark(ctx, "norm")
            return x, (delta if rows is None else NormedAhead(rows, next_norm))
        rows, delta = self._close(x, a, self.post_mixer_norm, self.ffn_norm, self.ffn_conv is not None)
        mark(ctx, "norm")
        if rows is None:
            h = self._read(ctx, self.ffn_norm, self.ffn_conv, x, delta, conv2_cache, False)
        else:
            h = self.ffn_conv.forward(ctx, rows, conv2_cache, out_dtype=self.rt.dtype) if self.ffn_conv is not None else rows
        mark(ctx, "conv" if self.ffn_conv is not None else "norm")
        d = self.ffn.forward(ctx, h)
        mark(ctx, "feed_forward")
        rows, delta = self._close(x, d, self.post_ffn_norm, next_norm, True)
        mark(ctx, "norm")
        return x, (delta if rows is None else NormedAhead(rows, next_norm))


@register_block("parallel")
class ParallelBlock(Block):
    """One norm, and a mixer and a feed-forward that both read its output and both add to the stream:

        h = norm(x);   x += mixer(h) + ffn(h)

    The feed-forward may be absent.  The mixer's output joins the stream at once (through its closing
    product where that can add itself, else by a sum kernel), the feed-forward's is handed on as `pending`;
    without a feed-forward the mixer's output is.

    The two sublayers depend on the norm's rows alone, so in steps of few rows, whose kernels are short and
    wait for one another, the feed-forward is queued on a second stream beside the mixer (also inside a
    captured step, where the two become branches of the graph); both streams meet before the block returns.
    Every use of the second stream begins by waiting for the first, after the norm that consumed what the
    second stream made last, so memory that either stream's allocator hands out again is no longer read by
    the other.  `LLOGOS_PARALLEL_STREAMS=0` keeps everything on one stream."""
    side_rows = 0 if os.environ.get("LLOGOS_PARALLEL_STREAMS", "1") == "0" else 64     # steps of up to so many rows use the second stream
    _side_streams = {}

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn: Optional[FeedForward] = None):
        self.mixer_norm, self.mixer, self.ffn = mixer_norm, mixer, ffn

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn] if self.ffn is not None else []

    def parts(self) -> List[Part]:
        return [p for p in (self.mixer_norm, self.mixer, self.ffn) if p is not None]

    def entry_norm(self) -> Optional[Norm]:
        return self.mixer_norm

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches):
        from ..ops import kernels as K
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        h = self.mixer_norm.forward(x, pending)
        mark(ctx, "norm")
        d = side = None
        if self.ffn is not None and h.shape[0] <= self.side_rows and (ctx is None or ctx.probe is None) and h.is_cuda:
            main = torch.cuda.current_stream(h.device)
            side = self._side_streams.get(h.device)
            if side is None:
                side = self._side_streams[h.device] = torch.cuda.Stream(device=h.device)
            side.wait_stream(main)                       # the norm's rows are there
            with torch.cuda.stream(side):
                d = self.ffn.forward(ctx, h)
        if self.mixer.adds_to_residual:
            a = self.mixer.forward(ctx, h, cache, residual=Residual(x, None))
        else:
            a = self.mixer.forward(ctx, h, cache)
        if isinstance(a, K.RowSquares):
            a = None                                     # the mixer's closing product has added itself to x
        mark(ctx, "mixer")
        if self.ffn is None:
            return x, a
        if a is not None:
            K.residual_add(x, K.sum_parts(a, None, torch.float32))
        if side is not None:
            torch.cuda.current_stream(h.device).wait_stream(side)
        else:
            d = self.ffn.forward(ctx, h)
        mark(ctx, "feed_forward")
        return x, d


@register_block("post_norm")
class PostNormBlock(Block):
    """The norm comes after the residual sum, and the stream itself is what the sublayers read:

        x <- mixer_norm(alpha * x + mixer(x));   x <- ffn_norm(alpha * x + ffn(x))

    The feed-forward (with its norm) may be absent.  The stream stays float32; each closing kernel
    (ops.kernels.post_norm: scaled sum, norm, weight) also leaves the new rows in the runtime's type for the
    sublayer that reads them next, and the block hands the last such rows on in place of a delta
    (`NormedAhead(rows, None)`: the stream is complete, and these are its own rows), which a block of this
    kind takes up and every norm ignores.  Norms that are not RMS norms with a row weight run their own
    kernel on the scaled sum instead."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None,
                 alpha: float = 1.0):
        if ffn is not None and ffn_norm is None:
            raise ValueError("a feed-forward comes with the norm behind its sum")
        # (a second norm without a feed-forward norms the scaled stream alone)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.alpha = float(alpha)

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn] if self.ffn is not None else []

    def parts(self) -> List[Part]:
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def entry_norm(self) -> Optional[Norm]:
        return None                      # the block's first reader takes the stream as it is

    def _close(self, x: torch.Tensor, out, norm: Norm) -> torch.Tensor:
        """x <- norm(alpha * x + out) in place; returns the new rows in the runtime's type."""
        from ..ops import kernels as K
        w = norm.row_weight()
        if w is not None and (out is None or isinstance(out, torch.Tensor)):
            return K.post_norm(x, out, self.alpha, w, norm.eps, self.rt.dtype)
        # any other norm: the stream scaled by a plain kernel, then the norm's own kernel, which adds `out`
        # (float32 rows where the norm can make them; a norm of the plain interface gives the runtime's type)
        import inspect
        K.scale_softcap(x, self.alpha)
        if "out_dtype" in inspect.signature(norm.forward).parameters:
            rows = norm.forward(x, out, out_dtype=torch.float32)
        else:
            rows = norm.forward(x, out)
        x.copy_(rows)
        return x if self.rt.is_f32 else K.sum_parts(x, None, self.rt.dtype)

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches):
        from ..ops import kernels as K
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        if isinstance(pending, NormedAhead) and pending.norm is None and pending.rows.dtype == self.rt.dtype:
            h = pending.rows                                  # the block before left the stream's rows
        else:
            if isinstance(pending, torch.Tensor):
                K.residual_add(x, K.sum_parts(pending, None, torch.float32))
            h = x if self.rt.is_f32 else K.sum_parts(x, None, self.rt.dtype)
        mark(ctx, "norm")
        a = self.mixer.forward(ctx, h, cache)
        mark(ctx, "mixer")
        h = self._close(x, a, self.mixer_norm)
        mark(ctx, "norm")
        if self.ffn_norm is not None:
            d = None
            if self.ffn is not None:
                d = self.ffn.forward(ctx, h)
                mark(ctx, "feed_forward")
            h = self._close(x, d, self.ffn_norm)
            mark(ctx, "norm")
        return x, (None if self.rt.is_f32 else NormedAhead(h, None))


@register_block("output_norm")
class OutputNormBlock(Block):
    """The norm stands on each sublayer's output alone, and the sublayers read the stream itself:

        x <- x + mixer_norm(mixer(x));   x <- x + ffn_norm(ffn(x))

    The feed-forward (with its norm) may be absent.  The stream stays float32; each closing kernel
    (ops.kernels.sandwich_norm: the output's norm and weight, the sum with the stream) also leaves the
    completed rows in the runtime's type for whoever reads them next, and the block hands the last such rows
    on in place of a delta (`NormedAhead(rows, None)`: the stream is complete, and these are its own rows),
    which a block that reads the stream itself takes up and every norm ignores.  Norms that are not RMS
    norms over the stream's width run their own kernel, and a sum kernel adds their rows."""

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Optional[Norm] = None, ffn: Optional[FeedForward] = None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with the norm on its output, or not at all")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def mixers(self) -> List[Mixer]:
        return [self.mixer]

    def feed_forwards(self) -> List[FeedForward]:
        return [self.ffn] if self.ffn is not None else []

    def parts(self) -> List[Part]:
        return [p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None]

    def entry_norm(self) -> Optional[Norm]:
        return None                      # the block's first reader takes the stream as it is

    def _close(self, x: torch.Tensor, out, norm: Norm) -> torch.Tensor:
        """x += norm(out) in place; returns the completed rows in the runtime's type."""
        from ..ops import kernels as K
        if isinstance(norm, RMSNorm) and x.shape[1] * 4 <= 65536:
            if self.rt.is_f32:
                K.sandwich_norm(x, out, norm.weight, None, norm.eps, torch.float32)
                return x
            return K.sandwich_norm(x, out, norm.weight, None, norm.eps, self.rt.dtype, plain_rows=True)
        import inspect
        a = out if (out.dim() == 2 and out.dtype == torch.float32) else K.sum_parts(out, None, torch.float32)
        if "out_dtype" in inspect.signature(norm.forward).parameters:
            rows = norm.forward(a, out_dtype=torch.float32)
        else:
            rows = norm.forward(a)
        K.residual_add(x, rows)
        return x if self.rt.is_f32 else K.sum_parts(x, None, self.rt.dtype)

    def forward(self, ctx: StepContext, x: torch.Tensor, pending, caches):
        from ..ops import kernels as K
        cache = caches[0] if isinstance(caches, (list, tuple)) else caches
        if isinstance(pending, NormedAhead) and pending.norm is None and pending.rows.dtype == self.rt.dtype:
            h = pending.rows                                  # the block before left the stream's rows
        else:
            if isinstance(pending, torch.Tensor):
                K.residual_add(x, K.sum_parts(pending, None, torch.float32))
            h = x if self.rt.is_f32 else K.sum_parts(x, None, self.rt.dtype)
        mark(ctx, "norm")
        a = self.mixer.forward(ctx, h, cache)
        mark(ctx, "mixer")
        h = self._close(x, a, self.mixer_norm)
        mark(ctx, "norm")
        if self.ffn is not None:
            d = self.ffn.forward(ctx, h)
            mark(ctx, "feed_forward")
            h = self._close(x, d, self.ffn_norm)
            mark(ctx, "norm")
        return x, (None if self.rt.is_f32 else NormedAhead(h, None))
