"""Python face of the HIP kernels: argument checks, then one call into the library.

Every function checks on the host that shapes, element types and devices match what the
kernel and its grid assume, and raises before anything is launched.  Tensors are torch
tensors used as device memory; launches go to torch's current stream.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
import os
from typing import Optional, Sequence, Tuple

import torch

from . import library
from ..cache.pages import HEAD_DIM_STEP, MAX_HEAD_DIM, PAGE_TOKENS      # the one definition; the library is checked against PAGE_TOKENS when loaded

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}
MAX_BANNED = 64             # ids one sampling call can set to -inf (kMaxBanned in csrc/sampling.hip)


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


def _lib():
    return library.load()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """torch's current stream of the current device, as the library takes it.  (The raw getter
    spares the ten microseconds a Stream object costs, once per launch.)"""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch._C._cuda_getDevice()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(*tensors) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel arguments must live on the GPU")
            _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _check(code: int, name: str) -> None:
    if code != 0:
        if code == -1:
            raise KernelError(f"{name}: bad argument")
        if code == -2:
            raise KernelError(f"{name}: size not supported")
        if code == -3:
            raise KernelError(f"{name}: larger than the library's fixed scratch array holds")
        raise KernelError(f"{name}: HIP error {code}")


def _i32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None:
        _need(t.dtype == torch.int32, f"{name} must be int32")


def _parts(t: Optional[torch.Tensor]) -> Tuple[int, int]:
    """(number of parts, elements between parts) of a product: [T, N] is one part,
    [P, T, N] are P partial sums that the consumer adds."""
    if t is None or t.dim() == 2:
        return 1, 0
    _need(t.dim() == 3, "a product must be [T, N] or [parts, T, N]")
    return t.shape[0], t.stride(0)


def _check_pools(k_pool: torch.Tensor, v_pool: Optional[torch.Tensor], n_kv_heads: int, head_dim: int, who: str) -> None:
    _need(head_dim % 16 == 0, f"{who}: head size {head_dim} is not a multiple of 16")
    _need(tuple(k_pool.shape[1:]) == (n_kv_heads, PAGE_TOKENS * head_dim),
          f"{who}: key pool must be [pages, kv_heads, {PAGE_TOKENS} * head_dim]")
    if v_pool is None:          # a cache whose values are part of its key rows
        _need(k_pool.is_contiguous(), f"{who}: the pool must be contiguous")
        return
    _need(tuple(v_pool.shape) == tuple(k_pool.shape),
          f"{who}: value pool must be [pages, kv_heads, {PAGE_TOKENS} * head_dim] like the key pool")
    _need(k_pool.is_contiguous() and v_pool.is_contiguous(), f"{who}: the pools must be contiguous")


# ----------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of `table` ([V, H], float32 or bfloat16) at int32 `ids`, times `scale`."""
    _dev(table, ids)
    _i32(ids, "ids")
    _need(table.dim() == 2 and ids.dim() == 1, "embed: table [V, H], ids [T]")
    T, H = ids.numel(), table.shape[1]
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _check(_lib().llogos_embed(_p(out), _p(table), _dt(table), _p(ids), T, H, ctypes.c_float(scale), _stream()), "embed")
    return out


def scale_softcap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """In place on float32 `x`: x * scale, then with cap > 0 bent to cap * tanh(x / cap)."""
    _dev(x)
    _need(x.dtype == torch.float32 and cap >= 0, "scale_softcap: float32 values, cap >= 0")
    if x.numel():
        _check(_lib().llogos_scale_softcap(_p(x), ctypes.c_longlong(x.numel()), ctypes.c_float(scale),
                                           ctypes.c_float(cap), _stream()), "scale_softcap")
    return x


def gather_i32(dst: torch.Tensor, src: torch.Tensor, rows: torch.Tensor) -> None:
    """dst[i] = src[rows[i]] for int32 vectors on the device."""
    _dev(dst, src, rows)
    _i32(dst, "dst"); _i32(src, "src"); _i32(rows, "rows")
    _need(dst.dim() == 1 and src.dim() == 1 and rows.dim() == 1 and dst.numel() == rows.numel()
          and dst.is_contiguous() and src.is_contiguous() and rows.is_contiguous(), "gather_i32: contiguous vectors, dst like rows")
    _check(_lib().llogos_gather_i32(_p(dst), _p(src), _p(rows), dst.numel(), src.numel(), _stream()), "gather_i32")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
            write_back: bool = True) -> torch.Tensor:
    """RMSNorm of the float32 residual stream `x` [T, H] with the pending `delta` ([T, H] or
    partial sums [parts, T, H]) added first (and written back to `x` when `write_back`).
    With `rows` only those rows are normed, into a compact output."""
    _dev(x, weight, delta, rows)
    _i32(rows, "rows")
    _need(x.dtype == torch.float32 and x.dim() == 2, "rmsnorm: x must be float32 [T, H]")
    T, H = x.shape
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "rmsnorm: weight must be float32 [H]")
    parts, part_stride = _parts(delta)
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == tuple(x.shape), "rmsnorm: delta must have x's shape")
    R = rows.numel() if rows is not None else T
    out = torch.empty((R, H), dtype=out_dtype, device=x.device)
    if R == 0:
        return out
    _check(_lib().llogos_rmsnorm(_p(out), _DT[out_dtype], _p(x), _p(delta), _dt(delta) if delta is not None else F32,
                                 parts, ctypes.c_longlong(part_stride),
                                 _p(rows), _p(weight), ctypes.c_float(eps), R, H, int(write_back), _stream()),
           "rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta: torch.Tensor) -> None:
    _dev(x, delta)
    _need(x.dtype == torch.float32 and delta.shape == x.shape, "residual_add: x float32, same shapes")
    _check(_lib().llogos_residual_add(_p(x), _p(delta), _dt(delta), ctypes.c_longlong(x.numel()), _stream()),
           "residual_add")


def layernorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
              delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None, write_back: bool = True) -> torch.Tensor:
    """(v - mean) / sqrt(variance + eps) * weight of the rows v = x + delta of the float32 stream x [T, H]
    (delta [T, H] or partial sums [parts, T, H]; with write_back the sum goes back to x); `rows` picks rows."""
    _dev(x, weight, delta, rows)
    _i32(rows, "rows")
    _need(x.dtype == torch.float32 and x.dim() == 2, "layernorm: the stream must be float32 [T, H]")
    T, H = x.shape
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "layernorm: weight must be float32 [H]")
    parts, part_stride = _parts(delta)
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == (T, H), "layernorm: delta must be [T, H] or [parts, T, H]")
        _need(parts == 1 or delta.dtype == torch.float32, "layernorm: parts must be float32")
    R = T if rows is None else rows.numel()
    out = torch.empty((R, H), dtype=out_dtype, device=x.device)
    if R:
        _check(_lib().llogos_layernorm(_p(out), _DT[out_dtype], _p(x), _p(delta), _dt(delta) if delta is not None else F32, parts,
                                       ctypes.c_longlong(part_stride), _p(rows), _p(weight), ctypes.c_float(eps), R, H,
                                       1 if write_back else 0, _stream()), "layernorm")
    return out


def add_sinusoid(x: torch.Tensor, positions: torch.Tensor, base: float = 10000.0) -> torch.Tensor:
    """In place on float32 x [T, W]: x[t, 2i] += sin(p_t * base^(-2i / W)), x[t, 2i + 1] += cos of the same."""
    _dev(x, positions)
    _i32(positions, "positions")
    _need(x.dtype == torch.float32 and x.dim() == 2 and positions.numel() == x.shape[0], "add_sinusoid: float32 [T, W] and T positions")
    _check(_lib().llogos_add_sinusoid(_p(x), _p(positions), x.shape[0], x.shape[1], ctypes.c_double(base), _stream()), "add_sinusoid")
    return x


def concat_rows(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype, delta: Optional[torch.Tensor] = None,
                write_back: bool = True) -> torch.Tensor:
    """[a + delta | b] row by row in `out_dtype`: float32 a [T, Wa] and b [T, Wb]; delta float32 [T, Wa] or
    partial sums [parts, T, Wa], added to a on the way (and written back to it)."""
    _dev(a, b, delta)
    _need(a.dtype == torch.float32 and b.dtype == torch.float32 and a.dim() == 2 and b.dim() == 2 and a.shape[0] == b.shape[0],
          "concat_rows: two float32 tensors of as many rows")
    parts, part_stride = _parts(delta)
    if delta is not None:
        _need(delta.dtype == torch.float32 and tuple(delta.shape[-2:]) == tuple(a.shape), "concat_rows: delta must be float32 like a")
    T, Wa, Wb = a.shape[0], a.shape[1], b.shape[1]
    out = torch.empty((T, Wa + Wb), dtype=out_dtype, device=a.device)
    _check(_lib().llogos_concat_rows(_p(out), _DT[out_dtype], _p(a), _p(delta), parts, ctypes.c_longlong(part_stride), _p(b), T, Wa, Wb,
                                     1 if write_back else 0, _stream()), "concat_rows")
    return out


def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias) with plain 32-bit FMAs."""
    _dev(w, bias)
    _need(a.is_cuda and a.dim() == 2 and a.stride(1) == 1, "gemm: a must be [M, K] with unit inner stride")
    M, K = a.shape
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    N = w.shape[0]
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    else:
        _need(out.shape == (M, N) and out.dtype == out_dtype and out.stride(1) == 1, "gemm: bad out")
    if M == 0:
        return out
    _check(_lib().llogos_gemm_generic(_p(out), _dt(out), _p(a), _dt(a), _p(w), _dt(w), _p(bias),
                                      M, N, K, a.stride(0), out.stride(0), _stream()), "gemm_generic")
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, amplitude: float = 1.0) -> torch.Tensor:
    """[T, half, 2] float32 (cos, sin) of positions[t] * inv_freq[i], computed in double, times `amplitude`."""
    _dev(positions, inv_freq)
    _i32(positions, "positions")
    _need(inv_freq.dtype == torch.float64 and inv_freq.dim() == 1, "rope_table: inv_freq must be float64 [half]")
    T, half = positions.numel(), inv_freq.numel()
    cs = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
    _check(_lib().llogos_rope_table(_p(cs), _p(positions), _p(inv_freq), T, half, ctypes.c_double(amplitude), _stream()), "rope_table")
    return cs


def qk_rope_cache(qkv: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                  n_heads: int, n_kv_heads: int, head_dim: int, rot: int, pairing: int,
                  q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], eps: float,
                  cs: torch.Tensor, k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor],
                  table: Optional[torch.Tensor], tok_seq: torch.Tensor, tok_pos: torch.Tensor) -> torch.Tensor:
    """From the fused projection rows [q | k | v] ([T, W] or partial sums [parts, T, W], plus
    `bias` [W]): per-head norm (optional) and rotation of q and k; q is returned
    [T, n_heads * head_dim] in `out_dtype`, k and v go to their cache pages."""
    _dev(qkv, bias, q_norm_w, k_norm_w, cs, k_pool, v_pool, table, tok_seq, tok_pos)
    _i32(tok_seq, "tok_seq"); _i32(tok_pos, "tok_pos"); _i32(table, "table")
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    _need(qkv.shape[-1] == width, f"qk_rope_cache: qkv must be [T, {width}]")
    _need(qkv.dtype == out_dtype or qkv.dtype == torch.float32, "qk_rope_cache: qkv must be float32 or the cache's type")
    _need(0 < head_dim <= MAX_HEAD_DIM, f"qk_rope_cache: head_dim {head_dim} not in 1..{MAX_HEAD_DIM}")
    _need(rot % 2 == 0 and 0 <= rot <= head_dim, "qk_rope_cache: rotary dimension must be even and <= head_dim")
    _need(cs.dtype == torch.float32 and cs.shape == (T, rot // 2, 2), "qk_rope_cache: rotary table shape")
    _need(tok_seq.numel() == T and tok_pos.numel() == T, "qk_rope_cache: per-token arrays must have T entries")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (width,), f"qk_rope_cache: bias must be float32 [{width}]")
    for wgt in (q_norm_w, k_norm_w):
        if wgt is not None:
            _need(wgt.dtype == torch.float32 and wgt.shape == (head_dim,), "qk_rope_cache: norm weight float32 [head_dim]")
    if n_kv_heads > 0:
        _need(k_pool is not None and v_pool is not None and table is not None, "qk_rope_cache: cache missing")
        _need(k_pool.dtype == out_dtype and v_pool.dtype == out_dtype, "qk_rope_cache: cache type differs")
        _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "qk_rope_cache")
        _need(table.dim() == 2, "qk_rope_cache: page table must be [batch, pages]")
    q_out = torch.empty((T, n_heads * head_dim), dtype=out_dtype, device=qkv.device)
    _check(_lib().llogos_qk_rope_cache(
        _p(qkv), _dt(qkv), parts, ctypes.c_longlong(part_stride), qkv.stride(-2), _p(bias), _p(q_out), _DT[out_dtype],
        n_heads, n_kv_heads, head_dim, rot, pairing,
        _p(q_norm_w), _p(k_norm_w), ctypes.c_float(eps), _p(cs), _p(k_pool), _p(v_pool),
        _p(table), table.stride(0) if table is not None else 0, _p(tok_seq), _p(tok_pos), T, _stream()),
        "qk_rope_cache")
    return q_out


GENERIC_MAX_HEAD_DIM = 1024      # the widest row the kernel for any shape takes (kMaxHeadDimGeneric)


def attention_generic(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor,
                      n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                      window: int = 0, sinks: int = 0, v_dim: Optional[int] = None,
                      head_sink: Optional[torch.Tensor] = None, softcap: float = 0.0,
                      gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of T query rows (row stride `q_stride` elements, heads first) over the
    paged cache; returns [T, n_heads * v_dim] in the cache's element type.  `v_pool` None:
    a value is the first `v_dim` dimensions of its key row.  `head_sink` float32 [n_heads]:
    a learned score per head that joins the softmax's denominator without a key or a value.
    With a value pool, values may have another width than keys (`v_dim`), and the pages' rows may be
    wider than either (the pools' last dimension says so).  `softcap` > 0 bends every score to
    softcap * tanh(score / softcap); `gate` float32 [T, >= n_heads] (a view of wider rows will do)
    multiplies head h's output by sigmoid(gate[t, h])."""
    _dev(k_pool, v_pool, table, tok_seq, tok_pos)
    _i32(tok_seq, "tok_seq"); _i32(tok_pos, "tok_pos"); _i32(table, "table")
    T = tok_seq.numel()
    _need(q.is_cuda and q.dtype == k_pool.dtype, "attention: q and cache types differ")
    _need(n_heads % n_kv_heads == 0, "attention: heads must be a multiple of kv heads")
    _need(0 < head_dim <= GENERIC_MAX_HEAD_DIM, f"attention: head_dim {head_dim} not in 1..{GENERIC_MAX_HEAD_DIM}")
    k_page_dim, v_page_dim = _page_dims(k_pool, v_pool, n_kv_heads, "attention")
    _need(k_page_dim >= head_dim, "attention: the key pages' rows are narrower than a head")
    _need(q_stride >= n_heads * head_dim and q.numel() >= (T - 1) * q_stride + n_heads * head_dim,
          "attention: q too small")
    v_dim = head_dim if v_dim is None else int(v_dim)
    _need(0 < v_dim <= (v_page_dim if v_pool is not None else head_dim) and v_dim <= GENERIC_MAX_HEAD_DIM,
          "attention: value width outside what the pages hold")
    if head_sink is not None:
        _dev(head_sink)
        _need(head_sink.dtype == torch.float32 and head_sink.shape == (n_heads,), "attention: head_sink must be float32 [n_heads]")
    gate_stride = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= n_heads
              and gate.stride(1) == 1, "attention: gate must be float32 [T, n_heads]")
        gate_stride = gate.stride(0) if T > 1 else max(n_heads, gate.stride(0))
    _need(softcap >= 0.0, "attention: softcap must not be negative")
    out = torch.empty((T, n_heads * v_dim), dtype=q.dtype, device=q.device)
    _check(_lib().llogos_attention_generic(
        _p(out), _p(q), _dt(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0),
        _p(tok_seq), _p(tok_pos), T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale),
        window, sinks, v_dim, _p(head_sink), k_page_dim, v_page_dim, ctypes.c_float(softcap), _p(gate), gate_stride,
        _stream()), "attention_generic")
    return out


def _page_dims(k_pool: torch.Tensor, v_pool: Optional[torch.Tensor], n_kv_heads: int, who: str) -> Tuple[int, int]:
    """(key row, value row) of the pools' pages, from their shapes [pages, kv_heads, PAGE_TOKENS * row]."""
    _need(k_pool.dim() == 3 and k_pool.shape[1] == n_kv_heads and k_pool.shape[2] % (PAGE_TOKENS * 8) == 0 and k_pool.is_contiguous(),
          f"{who}: key pool must be [pages, kv_heads, {PAGE_TOKENS} * row]")
    kd = k_pool.shape[2] // PAGE_TOKENS
    if v_pool is None:
        return kd, kd
    _need(v_pool.dim() == 3 and tuple(v_pool.shape[:2]) == tuple(k_pool.shape[:2]) and v_pool.shape[2] % (PAGE_TOKENS * 16) == 0
          and v_pool.is_contiguous() and v_pool.dtype == k_pool.dtype,
          f"{who}: value pool must be [pages, kv_heads, {PAGE_TOKENS} * row] like the key pool")
    return kd, v_pool.shape[2] // PAGE_TOKENS


def qkv_prepare(ctx, qkv: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype, n_heads: int, n_kv_heads: int,
                head_dim: int, v_dim: int, q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], eps: float,
                temp_coef: float, temp_every: int, k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor],
                table: Optional[torch.Tensor], writes: bool = True, cs: Optional[torch.Tensor] = None, rot: int = 0,
                pairing: int = 0, kv_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From projected rows [q | k | v | ...] (float32 [T, >= W] or partial sums [parts, T, >= W], plus `bias`
    [W], W = n_heads * head_dim + n_kv_heads * (head_dim + v_dim)): an RMS norm over the whole of q and of
    k where a weight is given ([n_heads * head_dim], [n_kv_heads * head_dim]), then the rotation of the first
    `rot` dimensions of every head of q and k by the table `cs` [T, rot / 2, 2] (pairing 0: dimension i with
    i + rot / 2, 1: 2i with 2i + 1), the query's factor 1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1);
    q comes back [T, n_heads * head_dim] in `out_dtype`, k and v go to their pages.  writes False: only q is
    made (the rows then need hold no more than q).  kv_rows: float32 [T, >= n_kv_heads * (head_dim + v_dim)] rows
    [k | v] in one part, for keys and values that were not projected together with q (qkv then holds q alone)."""
    _need(qkv.is_cuda and qkv.dtype == torch.float32 and qkv.stride(-1) == 1, "qkv_prepare: float32 rows on the GPU")
    _dev(bias, q_norm_w, k_norm_w, table, ctx.tok_seq, ctx.tok_pos)
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    Wq, Wk, Wv = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * v_dim
    width = Wq + ((Wk + Wv) if (writes and kv_rows is None) else 0)
    _need(qkv.shape[-1] >= width and T == ctx.n_tokens, f"qkv_prepare: rows of at least {width} values, one a token")
    kv_stride = 0
    if kv_rows is not None:
        _need(writes and kv_rows.is_cuda and kv_rows.dtype == torch.float32 and kv_rows.dim() == 2 and kv_rows.shape[0] == T
              and kv_rows.shape[1] >= Wk + Wv and kv_rows.stride(1) == 1, f"qkv_prepare: kv_rows must be float32 [T, >= {Wk + Wv}]")
        kv_stride = kv_rows.stride(0) if T > 1 else max(Wk + Wv, kv_rows.stride(0))
    _need(rot % 2 == 0 and 0 <= rot <= head_dim and pairing in (0, 1), "qkv_prepare: the rotated width must be even and within a head")
    if rot:
        _dev(cs)
        _need(cs is not None and cs.dtype == torch.float32 and tuple(cs.shape) == (T, rot // 2, 2), "qkv_prepare: rotary table shape")
    row_stride = qkv.stride(-2) if T > 1 else max(width, qkv.stride(-2))
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() >= width, f"qkv_prepare: bias must be float32 [{width}]")
    if q_norm_w is not None:
        _need(q_norm_w.dtype == torch.float32 and q_norm_w.shape == (Wq,), f"qkv_prepare: q norm weight float32 [{Wq}]")
    if k_norm_w is not None:
        _need(k_norm_w.dtype == torch.float32 and k_norm_w.shape == (Wk,), f"qkv_prepare: k norm weight float32 [{Wk}]")
    _need(temp_coef == 0.0 or temp_every >= 1, "qkv_prepare: the temperature's block must be at least one position")
    kd = vd = 0
    if writes:
        _need(k_pool is not None and v_pool is not None and table is not None, "qkv_prepare: cache missing")
        _i32(table, "table")
        _need(k_pool.dtype == out_dtype, "qkv_prepare: cache type differs")
        kd, vd = _page_dims(k_pool, v_pool, n_kv_heads, "qkv_prepare")
        _need(kd >= head_dim and vd >= v_dim and table.dim() == 2, "qkv_prepare: pages narrower than the heads")
    q_out = torch.empty((T, Wq), dtype=out_dtype, device=qkv.device)
    _check(_lib().llogos_qkv_prepare(
        _p(qkv), parts, ctypes.c_longlong(part_stride), row_stride, _p(bias), _p(q_out), _DT[out_dtype], n_heads,
        n_kv_heads if writes else 0, head_dim, v_dim, kd, vd, _p(q_norm_w), _p(k_norm_w), ctypes.c_float(eps),
        ctypes.c_float(temp_coef), int(temp_every), _p(cs) if rot else None, int(rot), int(pairing), _p(k_pool) if writes else None, _p(v_pool) if writes else None,
        _p(table) if writes else None, table.stride(0) if (writes and table is not None) else 0, _p(ctx.tok_seq), _p(ctx.tok_pos),
        _p(kv_rows), kv_stride, T, _stream()), "qkv_prepare")
    return q_out


def swiglu(gu: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """silu(gate) * up from fused rows [gate | up] ([T, 2 I] or partial sums [parts, T, 2 I])."""
    _dev(gu)
    parts, part_stride = _parts(gu)
    _need(gu.shape[-1] % 2 == 0, "swiglu: rows must be [gate | up]")
    out_dtype = out_dtype or gu.dtype
    _need(gu.dtype == out_dtype or gu.dtype == torch.float32, "swiglu: input must be float32 or the output's type")
    T, I = gu.shape[-2], gu.shape[-1] // 2
    out = torch.empty((T, I), dtype=out_dtype, device=gu.device)
    _check(_lib().llogos_swiglu(_p(out), _DT[out_dtype], _p(gu), _dt(gu), parts, ctypes.c_longlong(part_stride),
                                T, I, _stream()), "swiglu")
    return out


def sum_parts(product: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype) -> torch.Tensor:
    """One plain [T, N] tensor of `out_dtype` from a product that may come in parts, plus bias."""
    _dev(product, bias)
    parts, part_stride = _parts(product)
    if parts == 1 and bias is None and product.dtype == out_dtype:
        return product if product.dim() == 2 else product[0]
    _need(parts == 1 or product.dtype == torch.float32, "sum_parts: parts must be float32")
    T, N = product.shape[-2:]
    out = torch.empty((T, N), dtype=out_dtype, device=product.device)
    _check(_lib().llogos_sum_parts(_p(out), _DT[out_dtype], _p(product), _dt(product), parts, ctypes.c_longlong(part_stride),
                                   _p(bias), T, N, _stream()), "sum_parts")
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """int32 index of the first maximum of each row of float32 logits."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits must be float32 [R, V]")
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    _check(_lib().llogos_argmax(_p(out), _p(logits), R, V, _stream()), "argmax")
    return out


# ----------------------------------------------------------------------------
# parts with a fixed-size state per sequence
# ----------------------------------------------------------------------------
MAX_CONV_TAPS = 16
ACTIVATIONS = {"tanh": 0, "silu": 1, "gelu_tanh": 2, "xielu": 3, "relu2": 4}


def causal_conv(ctx, h: torch.Tensor, w: torch.Tensor, state: torch.Tensor, out_dtype: torch.dtype,
                add_input: bool = True, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """h + conv(h) over time, channel by channel (conv(h) alone with add_input False; `bias` float32 [W] is
    added to every output): h float32 [T, W] (the step's rows, one sequence after the other; it may be W
    columns of wider rows), w float32 [W, taps] whose last tap multiplies the present token, state float32
    [slots, >= taps - 1, W]: a sequence's last taps - 1 inputs in the first rows of its slot (rows behind
    them are another mechanism's), read for the rows before the step's first and brought up to date."""
    _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1, "causal_conv: h must be rows on the GPU")
    _dev(w, bias, ctx.slots, ctx.tok_seq, ctx.tok_pos, ctx.cu_dev)
    _need(h.dtype == torch.float32, "causal_conv: h must be float32 [T, W]")
    T, W = h.shape
    _need(w.dtype == torch.float32 and w.dim() == 2 and w.shape[0] == W and 1 <= w.shape[1] <= MAX_CONV_TAPS,
          f"causal_conv: w must be float32 [W, taps] with at most {MAX_CONV_TAPS} taps")
    taps = w.shape[1]
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 3 and state.shape[1] >= max(taps - 1, 0)
          and state.shape[2] == W and (state.shape[1] == 0 or (state.stride(2) == 1 and state.stride(1) == W)),
          "causal_conv: state must be float32 [slots, >= taps - 1, W] with dense rows")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (W,), "causal_conv: bias must be float32 [W]")
    _need(T == ctx.n_tokens and ctx.tok_seq.numel() == T and ctx.tok_pos.numel() == T, "causal_conv: one row a token of the step")
    _need(ctx.cu_dev is not None or T == ctx.batch, "causal_conv: a step of several tokens a sequence needs the token offsets")
    out = torch.empty((T, W), dtype=out_dtype, device=h.device)
    slot_stride = 0                      # (a state without rows: one tap reads no row before the present one)
    if state.shape[1] > 0:
        slot_stride = state.stride(0) if state.shape[0] > 1 else state.shape[1] * W
    _check(_lib().llogos_causal_conv(_p(out), _DT[out_dtype], _p(h), _p(w), _p(state), _p(ctx.slots), _p(ctx.tok_seq),
                                     _p(ctx.tok_pos), _p(ctx.cu_dev), T, ctx.batch, W, h.stride(0) if T > 1 else max(W, h.stride(0)),
                                     taps, 1 if add_input else 0, _p(bias), ctypes.c_longlong(slot_stride), _stream()), "causal_conv")
    return out


def token_shift(ctx, h: torch.Tensor, mu: torch.Tensor, prev: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[n, T, W]: h + (row before - h) * mu[s] for each of the n rows of mu; the row before a
    sequence's first row of the step is prev[slot] (`prev` float32 [slots, W], maybe a column
    range of a wider state tensor; it is read, not written)."""
    _dev(h, mu, ctx.slots, ctx.tok_seq, ctx.cu_dev)
    _need(h.dtype == torch.float32 and h.dim() == 2, "token_shift: h must be float32 [T, W]")
    T, W = h.shape
    _need(mu.dtype == torch.float32 and mu.dim() == 2 and mu.shape[1] == W, "token_shift: mu must be float32 [n, W]")
    _need(prev.is_cuda and prev.dtype == torch.float32 and prev.dim() == 2 and prev.shape[1] == W and prev.stride(1) == 1,
          "token_shift: prev must be float32 [slots, W]")
    _need(ctx.cu_dev is not None or T == ctx.batch, "token_shift: a step of several tokens a sequence needs the token offsets")
    n = mu.shape[0]
    out = torch.empty((n, T, W), dtype=out_dtype, device=h.device)
    _check(_lib().llogos_token_shift(_p(out), _DT[out_dtype], _p(h), _p(mu), _p(prev), ctypes.c_longlong(prev.stride(0)),
                                     _p(ctx.slots), _p(ctx.tok_seq), _p(ctx.cu_dev), T, W, n, _stream()), "token_shift")
    return out


def wkv_scan(ctx, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, d: torch.Tensor, gate: torch.Tensor,
             w0: torch.Tensor, u: torch.Tensor, g: torch.Tensor, eps: float, state: torch.Tensor, n_heads: int,
             dim: int, h_in: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """The recurrence S <- diag(w) S + k v^T with output (S + diag(u) k v^T)^T r per head, the
    per-head RMS scale, weight g and silu(gate), over the step's rows of each sequence in turn.
    r, k, v, d, gate: float32 [T, heads * dim] (w = exp(-exp(d + w0))), or partial sums [parts, T, heads * dim] of
    products split along k (r, k, v, gate with one split, d with its own); state float32
    [slots, heads * dim * dim + W]: each head's S as [value channel][key channel], then the
    last mixer input row, which this kernel replaces by h_in's last row of each sequence."""
    HD = n_heads * dim
    _dev(r, k, v, d, gate, w0, u, g, state, h_in, ctx.slots, ctx.cu_dev)
    for t, name in ((r, "r"), (k, "k"), (v, "v"), (d, "d"), (gate, "gate")):
        _need(t.dtype == torch.float32 and t.dim() in (2, 3) and tuple(t.shape[-2:]) == (ctx.n_tokens, HD),
              f"wkv_scan: {name} must be float32 [T, heads * dim] or parts of it")
    parts, part_stride = _parts(r)
    for t in (k, v, gate):
        _need(_parts(t) == (parts, part_stride), "wkv_scan: r, k, v and gate must be split alike")
    d_parts, d_part_stride = _parts(d)
    for t, name in ((w0, "w0"), (u, "u"), (g, "g")):
        _need(t.dtype == torch.float32 and t.numel() == HD, f"wkv_scan: {name} must be float32 [heads * dim]")
    W = h_in.shape[1]
    _need(h_in.dtype == torch.float32 and h_in.shape == (ctx.n_tokens, W), "wkv_scan: h_in must be float32 [T, W]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == HD * dim + W, "wkv_scan: state must be float32 [slots, heads * dim * dim + W]")
    _need(ctx.cu_dev is not None or ctx.n_tokens == ctx.batch, "wkv_scan: a step of several tokens a sequence needs the token offsets")
    _need(6 * dim * 4 <= 65536, f"wkv_scan: head size {dim} is too large")
    y = torch.empty((ctx.n_tokens, HD), dtype=out_dtype, device=r.device)
    rows, col_blocks, n_seg = scan_plan(ctx.batch, n_heads, dim, None if ctx.is_decode else
                                        max(ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)))
    o_raw = torch.empty((ctx.n_tokens, HD), dtype=torch.float32, device=r.device) if col_blocks > 1 else None
    seg_len, seg_state, seg_decay = 0, None, None
    if n_seg > 1:
        longest = max(ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch))
        seg_len = -(-(-(-longest // n_seg)) // 16) * 16                  # whole chunks of the kernel
        seg_state = torch.empty((ctx.batch, n_seg, n_heads, dim, dim), dtype=torch.float32, device=r.device)
        seg_decay = torch.empty((ctx.batch, n_seg, n_heads, dim), dtype=torch.float32, device=r.device)
    _check(_lib().llogos_wkv_scan(_p(y), _DT[out_dtype], _p(r), _p(k), _p(v), _p(d), _p(gate), HD, parts, ctypes.c_longlong(part_stride),
                                  d_parts, ctypes.c_longlong(d_part_stride), _p(w0), _p(u), _p(g),
                                  ctypes.c_float(eps), _p(state), ctypes.c_longlong(state.stride(0)), ctypes.c_longlong(HD * dim),
                                  _p(h_in), W, _p(ctx.slots), _p(ctx.cu_dev), ctx.batch, n_heads, dim, ctx.n_tokens, col_blocks,
                                  _p(o_raw), n_seg, seg_len, _p(seg_state), _p(seg_decay), rows, _stream()), "wkv_scan")
    return y


SCAN_COLUMN_BLOCKS = 0       # 0: chosen by the step; 1, 2, 4, ... force the number of blocks a head (tests)
SCAN_SEGMENTS = 0            # 0: chosen by the step; 1, 2, 3, ... force the number of segments of a prompt (tests)
SCAN_ROWS = 0                # 0: chosen by the step; 4 or 16 force the rows of the state a thread (tests)


def scan_plan(batch: int, n_heads: int, dim: int, longest: Optional[int], n_cus: Optional[int] = None) -> Tuple[int, int, int]:
    """(rows of the state a thread, blocks a head, segments a prompt) for the recurrence; `longest` is the most
    tokens a sequence brings (None: a single-token step).  Measured on the MI355X (64 heads of 64, one prompt of
    2,048 tokens): a block a head with 4 rows a thread 1,014 us, its columns over 4 blocks 550 us (a chain of
    2,048 dependent steps of 270 ns, whatever else is done); cut into 4 to 16 segments that run side by side
    (each twice: once for its end state from zero, once for its outputs from its true initial state) 455 us, no
    longer bound by the chain but by the instructions a token costs a thread, of which with 4 rows a thread two
    thirds fetch r, k and the decay and add up the parts; hence 16 rows a thread wherever the blocks fill the
    machine without the finer split.
    Segments: as many as bring the waves to about six a SIMD, of at least 128 tokens, at most 16."""
    n_cus = n_cus or compute_units()
    simds = 4 * n_cus
    wide = dim % 16 == 0 and dim <= 256                              # 16 rows a thread tile the head exactly
    waves16 = batch * n_heads * max(1, (dim * max(1, dim // 16) + 63) // 64) if wide else 0
    n_seg = 1
    if longest is not None:
        base = waves16 if wide else batch * n_heads * max(1, (dim * 16 + 63) // 64)
        n_seg = max(1, min(16, longest // 128, -(-(6 * simds) // max(1, base))))
    if SCAN_SEGMENTS and longest is not None:
        n_seg = SCAN_SEGMENTS
    if SCAN_COLUMN_BLOCKS and longest is not None:
        return 4, SCAN_COLUMN_BLOCKS, n_seg
    if SCAN_ROWS == 16 or (wide and waves16 * n_seg >= 2 * simds and not SCAN_ROWS):
        return 16, 1, n_seg
    blocks, pairs = 1, batch * n_heads * n_seg
    if longest is not None and longest >= 64:
        while blocks * 2 * pairs <= n_cus and dim // (blocks * 2) >= 16 and dim % (blocks * 2) == 0:
            blocks *= 2
    return 4, blocks, n_seg


def sandwich_norm(x: torch.Tensor, a: torch.Tensor, post_w: torch.Tensor, next_w: Optional[torch.Tensor], eps: float,
                  out_dtype: torch.dtype, plain_rows: bool = False) -> Optional[torch.Tensor]:
    """x += rmsnorm(a) * post_w in place (x the float32 stream [T, H]; a [T, H] or float32 partial sums
    [parts, T, H]), and, with next_w, the rows rmsnorm(x) * next_w of the completed stream in `out_dtype`;
    with plain_rows (and no next_w) the completed rows themselves in `out_dtype`."""
    _dev(x, a, post_w, next_w)
    _need(x.dtype == torch.float32 and x.dim() == 2, "sandwich_norm: x must be float32 [T, H]")
    T, H = x.shape
    parts, part_stride = _parts(a)
    _need(tuple(a.shape[-2:]) == (T, H) and (parts == 1 or a.dtype == torch.float32), "sandwich_norm: a must have x's shape")
    _need(post_w.dtype == torch.float32 and post_w.shape == (H,), "sandwich_norm: weights must be float32 [H]")
    _need(next_w is None or (next_w.dtype == torch.float32 and next_w.shape == (H,)), "sandwich_norm: weights must be float32 [H]")
    _need(not (plain_rows and next_w is not None), "sandwich_norm: plain rows or the next norm's rows, not both")
    _need(H * 4 <= 65536, "sandwich_norm: rows of more than 16,384 values")
    h = torch.empty((T, H), dtype=out_dtype, device=x.device) if (next_w is not None or plain_rows) else None
    if T:
        _check(_lib().llogos_sandwich_norm(_p(x), _p(a), _dt(a), parts, ctypes.c_longlong(part_stride), _p(post_w), _p(next_w),
                                           _p(h), _DT[out_dtype], ctypes.c_float(eps), T, H, _stream()), "sandwich_norm")
    return h


def activation(x: torch.Tensor, kind: str, out_dtype: torch.dtype, a: float = 0.0, b: float = 0.0,
               cols: Optional[int] = None) -> torch.Tensor:
    """act(x) element by element; x [T, N] or float32 partial sums [parts, T, N] that are added first.
    kinds: tanh, silu, gelu_tanh, xielu (z > 0: a z^2 + z / 2; z <= 0: b (exp(z) - 1 - z) + z / 2), relu2
    (the square of max(z, 0)).  cols: only the first `cols` values of every row are taken (the result is
    [T, cols]): a product whose rows hold something else behind them."""
    _dev(x)
    _need(kind in ACTIVATIONS, f"activation: unknown kind '{kind}'; known: {sorted(ACTIVATIONS)}")
    parts, part_stride = _parts(x)
    _need(parts == 1 or x.dtype == torch.float32, "activation: parts must be float32")
    T, N = x.shape[-2:]
    C = N if cols is None else int(cols)
    _need(0 < C <= N, "activation: cols outside 1..N")
    out = torch.empty((T, C), dtype=out_dtype, device=x.device)
    if out.numel():
        _check(_lib().llogos_activation(_p(out), _DT[out_dtype], _p(x), _dt(x), parts, ctypes.c_longlong(part_stride),
                                        ctypes.c_longlong(T * C), ACTIVATIONS[kind], ctypes.c_float(a), ctypes.c_float(b),
                                        0 if C == N else C, N, _stream()),
               "activation")
    return out


# ----------------------------------------------------------------------------
# experts chosen by a table over token ids
# ----------------------------------------------------------------------------
MOE_MAX_EXPERTS = 1024
MOE_FEW_PAIRS = 256          # up to so many (token, choice) pairs a step the experts' product streams the matrices in tiles of 16 rows
MOE_PRODUCT = "auto"         # "auto": chosen by the step; "plain", "few", "tiles64", "tiles128" force a form (tests)


def moe_route(ids: Optional[torch.Tensor], table: torch.Tensor, n_experts: int):
    """(order, seg, where) int32 on the device: the step's (token, choice) pairs t * top + j sorted by
    their expert table[ids[t], j], the experts' segments in that order (n_experts + 1 offsets) and each
    pair's place in it.  ids None: table [T, top] holds each token's own choices (a router's)."""
    _dev(ids, table)
    _i32(ids, "ids"); _i32(table, "table")
    _need(table.dim() == 2 and 0 < n_experts <= MOE_MAX_EXPERTS, f"moe_route: table [rows, top], at most {MOE_MAX_EXPERTS} experts")
    _need(ids is None or ids.dim() == 1, "moe_route: ids [T]")
    T, top = (ids.numel() if ids is not None else table.shape[0]), table.shape[1]
    buf = torch.empty(2 * T * top + n_experts + 1, dtype=torch.int32, device=table.device)
    order, where, seg = buf[:T * top], buf[T * top:2 * T * top], buf[2 * T * top:]
    _check(_lib().llogos_moe_route(_p(ids), _p(table), T, top, n_experts, _p(order), _p(seg), _p(where), _stream()), "moe_route")
    return order, seg, where


def moe_router(h: torch.Tensor, router_w: torch.Tensor, correction: Optional[torch.Tensor], n_groups: int, keep: int, top: int,
               scale: float):
    """A router's choice for every row of h [T, K] (any storage type): logits z = h . router_w^T in 32-bit
    (router_w float32 [E, K]), s = softmax(z) over all E outputs, the choice's scores s + correction (float32 [E]
    or None), of which only those in the `keep` best of n_groups equal groups of neighbouring outputs (a group's
    score is its largest) can be chosen; the `top` largest are chosen (the lowest index among equals).
    Returns (choice int32 [T, top], weight float32 [T, top]) with weight = s[choice] / (their sum + 1e-20) * scale."""
    _dev(router_w, correction)
    _need(h.is_cuda and h.dim() == 2 and h.stride(1) == 1, "moe_router: rows [T, K] on the GPU")
    _need(router_w.dtype == torch.float32 and router_w.dim() == 2 and router_w.shape[1] == h.shape[1], "moe_router: router_w must be float32 [E, K]")
    T, Kk = h.shape
    E = router_w.shape[0]
    _need(0 < top <= E <= MOE_MAX_EXPERTS, f"moe_router: top within 1..E, at most {MOE_MAX_EXPERTS} outputs")
    _need(correction is None or (correction.dtype == torch.float32 and correction.shape == (E,)), "moe_router: correction must be float32 [E]")
    n_groups, keep = max(1, int(n_groups)), int(keep)
    if n_groups > 1:
        _need(E % n_groups == 0 and keep >= 1 and min(keep, n_groups) * (E // n_groups) >= top,
              "moe_router: equal groups, and the kept ones must hold at least `top` outputs")
    z = torch.empty((T, E), dtype=torch.float32, device=h.device)
    _check(_lib().llogos_moe_router_logits(_p(z), _p(h), _dt(h), h.stride(0) if T > 1 else max(Kk, h.stride(0)), _p(router_w),
                                           T, E, Kk, _stream()), "moe_router_logits")
    choice = torch.empty((T, top), dtype=torch.int32, device=h.device)
    weight = torch.empty((T, top), dtype=torch.float32, device=h.device)
    _check(_lib().llogos_moe_router_choose(_p(z), _p(correction), T, E, n_groups, keep, top, ctypes.c_float(scale), _p(choice),
                                           _p(weight), _stream()), "moe_router_choose")
    return choice, weight


def moe_combine_weighted(y: torch.Tensor, where: torch.Tensor, choice: torch.Tensor, weight: torch.Tensor, n_real: int,
                         h: torch.Tensor, shared: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, W]: sum_j weight[t, j] * row_j + shared[t], where row_j is the pair's row y[where[t * top + j]]
    when choice[t, j] < n_real and the token's own row h[t] otherwise (a router output that has no matrices and
    returns its input).  y float32 [T * top, W]; h [T, W] of any storage type; shared float32 [T, W] or parts."""
    _dev(y, where, choice, weight)
    _i32(where, "where"); _i32(choice, "choice")
    _need(choice.dim() == 2 and weight.shape == choice.shape and weight.dtype == torch.float32, "moe_combine_weighted: choice and weight [T, top]")
    T, top = choice.shape
    _need(y.dtype == torch.float32 and y.dim() == 2 and y.shape[0] == T * top and where.numel() == T * top, "moe_combine_weighted: y float32 [T * top, W]")
    W = y.shape[1]
    _need(h.is_cuda and h.dim() == 2 and h.shape == (T, W) and h.stride(1) == 1, "moe_combine_weighted: h must be [T, W]")
    parts, part_stride = 1, 0
    if shared is not None:
        _dev(shared)
        parts, part_stride = _parts(shared)
        _need(shared.dtype == torch.float32 and tuple(shared.shape[-2:]) == (T, W), "moe_combine_weighted: shared rows float32 [T, W]")
    out = torch.empty((T, W), dtype=torch.float32, device=y.device)
    _check(_lib().llogos_moe_combine_weighted(_p(out), _p(y), _p(where), _p(choice), _p(weight), top, int(n_real), _p(h), _dt(h),
                                              h.stride(0) if T > 1 else max(W, h.stride(0)), _p(shared), parts,
                                              ctypes.c_longlong(part_stride), T, W, _stream()), "moe_combine_weighted")
    return out


def moe_product(a: torch.Tensor, w: torch.Tensor, order: torch.Tensor, seg: torch.Tensor, top: int, gather: bool,
                out_dtype: torch.dtype, relu2: bool = False, scale: float = 1.0, gated: bool = False) -> torch.Tensor:
    """[P, N]: sorted row r, which belongs to the expert e whose segment holds it, is a_row(r) . w[e]^T, with
    a_row(r) = a[order[r] // top] (gather: a holds the step's token rows) or a[r] (a is sorted already);
    w [E, N, K]; relu2 squares max(., 0) in the epilogue, scale multiplies the result.  gated: the rows of
    w[e] are gate and up rows in turn (gate 0, up 0, gate 1, ...) and the result is [P, N / 2], column i
    silu(gate_i sum) * (up_i sum).  `seg` may hold more segments than w has experts: rows in those belong
    to choices without a matrix and are left unwritten."""
    _dev(a, w, order, seg)
    _i32(order, "order"); _i32(seg, "seg")
    _need(a.dim() == 2 and w.dim() == 3 and a.shape[1] == w.shape[2] and seg.numel() >= w.shape[0] + 1, "moe_product: a [M, K], w [E, N, K]")
    _need(a.dtype == w.dtype, "moe_product: rows and matrices of one type")
    _need(not (relu2 and gated), "moe_product: one epilogue at a time")
    E, N, Kk = w.shape
    P = order.numel()
    _need(gather or a.shape[0] == P, "moe_product: sorted rows must be as many as pairs")
    _need(not gather or a.shape[0] * top == P, "moe_product: token rows times choices must be the pairs")
    _need(not gated or N % 2 == 0, "moe_product: gate and up rows in turn make an even number of rows")
    act = 2 if gated else (1 if relu2 else 0)
    out = torch.empty((P, N // 2 if gated else N), dtype=out_dtype, device=a.device)
    if a.dtype == torch.bfloat16 and MOE_PRODUCT != "plain" and a.stride(1) == 1:
        # on the matrix cores: tiles of 16 sorted rows straight from memory for steps of few rows, tiles of 64 or
        # 128 rows through LDS where an expert's segment is long enough on average to fill them
        form = 0 if P <= MOE_FEW_PAIRS else (2 if P >= 96 * E else 1)
        if MOE_PRODUCT in ("few", "tiles64", "tiles128"):
            form = ("few", "tiles64", "tiles128").index(MOE_PRODUCT)
        code = _lib().llogos_moe_product_bf16(_p(out), _DT[out_dtype], _p(a), _p(w), _p(order), _p(seg), E, top, 1 if gather else 0,
                                              P, N, Kk, a.stride(0), act, ctypes.c_float(scale), form, _stream())
        if code != -2:
            _check(code, "moe_product")
            return out
    _check(_lib().llogos_moe_product(_p(out), _DT[out_dtype], _p(a), _dt(a), _p(w), _dt(w), _p(order), _p(seg), E, top,
                                     1 if gather else 0, P, N, Kk, a.stride(0), act, ctypes.c_float(scale), _stream()),
           "moe_product")
    return out


def moe_combine(y: torch.Tensor, where: torch.Tensor, top: int, shared: Optional[torch.Tensor] = None,
                gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, W]: the mean of each token's pair rows y[where[t * top + j]], plus its shared row times
    sigmoid(gate[t]).  shared float32 [T, W] or parts [parts, T, W]; gate a float32 column [T, 1] (a view of
    one column of wider rows will do) or parts [parts, T, 1] of it."""
    _dev(y, where)
    _i32(where, "where")
    _need(y.dtype == torch.float32 and y.dim() == 2 and where.numel() == y.shape[0] and y.shape[0] % top == 0, "moe_combine: y float32 [T * top, W]")
    T, W = y.shape[0] // top, y.shape[1]
    parts, part_stride = 1, 0
    if shared is not None:
        _dev(shared)
        parts, part_stride = _parts(shared)
        _need(shared.dtype == torch.float32 and tuple(shared.shape[-2:]) == (T, W), "moe_combine: shared rows float32 [T, W]")
    g_parts, g_part_stride, g_stride = 1, 0, 1
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() in (2, 3) and tuple(gate.shape[-2:]) == (T, 1),
              "moe_combine: gate float32 [T, 1]")
        g_stride = gate.stride(-2) if T > 1 else 1
        if gate.dim() == 3:
            g_parts, g_part_stride = gate.shape[0], gate.stride(0)
    out = torch.empty((T, W), dtype=torch.float32, device=y.device)
    _check(_lib().llogos_moe_combine(_p(out), _p(y), _p(where), top, _p(shared), parts, ctypes.c_longlong(part_stride), _p(gate),
                                     g_stride, g_parts, ctypes.c_longlong(g_part_stride), T, W, _stream()), "moe_combine")
    return out


# ----------------------------------------------------------------------------
# attention through a latent
# ----------------------------------------------------------------------------
def latent_prepare(ctx, kv: torch.Tensor, qfull: torch.Tensor, q_out: torch.Tensor, norm_w: torch.Tensor, eps: float,
                   cs: Optional[torch.Tensor], k_pool: torch.Tensor, v_pool: Optional[torch.Tensor], table: torch.Tensor,
                   n_heads: int, dim: int, rot: int, rot_dims: int, rank: int, c_out: Optional[torch.Tensor] = None) -> None:
    """From kv float32 [T, rank + rot] and qfull float32 [T, heads * (dim + rot)]: the normed latent and
    the rotated shared key part go to the token's key row in the cache ([rank | rot | zeros]); each
    head's rotated query part goes to q_out[t, h, rank:] ([T, heads, hd], hd the cache's row width).  With a
    value pool the latent is also stored as the token's value row, and with c_out ([T, rank] of the cache's type)
    as plain rows."""
    _dev(q_out, norm_w, cs, k_pool, v_pool, table, ctx.tok_seq, ctx.tok_pos)
    _i32(table, "table")
    T = ctx.n_tokens
    hd = q_out.shape[-1]
    # (kv and qfull may be columns of wider rows)
    _need(kv.is_cuda and kv.dtype == torch.float32 and kv.shape == (T, rank + rot) and kv.stride(1) == 1,
          "latent_prepare: kv must be float32 [T, rank + rot]")
    _need(qfull.is_cuda and qfull.dtype == torch.float32 and qfull.shape == (T, n_heads * (dim + rot)) and qfull.stride(1) == 1,
          "latent_prepare: q must be float32 [T, heads * (dim + rot)]")
    _need(q_out.shape == (T, n_heads, hd) and q_out.dtype == k_pool.dtype, "latent_prepare: q_out must be [T, heads, hd] of the cache's type")
    _need(hd % 16 == 0 and hd >= rank + rot, "latent_prepare: the cache's row is too narrow")
    _check_pools(k_pool, v_pool, 1, hd, "latent_prepare")
    _need(v_pool is None or v_pool.dtype == k_pool.dtype, "latent_prepare: the pools' types differ")
    _need(norm_w.dtype == torch.float32 and norm_w.shape == (rank,), "latent_prepare: norm weight must be float32 [rank]")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= rot, "latent_prepare: rotated dimensions must be even and within rot")
    if rot_dims:
        _need(cs is not None and cs.dtype == torch.float32 and cs.shape == (T, rot_dims // 2, 2), "latent_prepare: rotary table shape")
    _need(table.dim() == 2, "latent_prepare: page table must be [batch, pages]")
    if c_out is not None:
        _dev(c_out)
        _need(c_out.shape == (T, rank) and c_out.dtype == k_pool.dtype, "latent_prepare: c_out must be [T, rank] of the cache's type")
    ld = lambda t_, least: t_.stride(0) if T > 1 else max(least, t_.stride(0))
    _check(_lib().llogos_latent_prepare(_p(kv), ld(kv, rank + rot), _p(qfull), ld(qfull, n_heads * (dim + rot)), _p(q_out), _dt(q_out), _p(norm_w),
                                        ctypes.c_float(eps), _p(cs), _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(ctx.tok_seq),
                                        _p(ctx.tok_pos), T, n_heads, dim, rot, rot_dims, rank, hd, _p(c_out), _stream()), "latent_prepare")


LATENT_MFMA_MAX_ROW = 576


def latent_attention_mfma(ctx, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, table: torch.Tensor,
                          n_heads: int, row: int, dv: int, scale: float, head_sink: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """bfloat16 attention over a latent cache on the matrix cores: q [T, heads, row], key rows and value rows
    (the latent in the value pages' order) in pools [pages, 1, 64 * row]; returns [T, heads, dv], or None
    for rows wider than the kernel takes.  Single-token steps share a sequence's pages out over several
    blocks (chosen from the batch and the longest context the step may have) and merge."""
    if q.dtype != torch.bfloat16 or row > LATENT_MFMA_MAX_ROW:
        return None
    T = ctx.n_tokens
    _dev(q, k_pool, v_pool, table, head_sink, ctx.tok_pos, ctx.cu_dev)
    _i32(table, "table")
    _need(q.shape == (T, n_heads, row) and row % 16 == 0 and 0 < dv <= row, "latent attention: q must be [T, heads, row]")
    _check_pools(k_pool, v_pool, 1, row, "latent attention")
    _need(k_pool.dtype == torch.bfloat16 and v_pool is not None and v_pool.dtype == torch.bfloat16, "latent attention: bfloat16 pools")
    if head_sink is not None:
        _need(head_sink.dtype == torch.float32 and head_sink.shape == (n_heads,), "latent attention: head_sink must be float32 [heads]")
    _need(table.dim() == 2 and table.shape[0] == ctx.batch, "latent attention: one table row a sequence")
    lib = _lib()
    splits, pps, ws, floats = 1, max(1, table.shape[1]), None, 0
    if ctx.is_decode:
        _need(T == ctx.batch, "latent attention: a single-token step has one token a sequence")
        n_tiles = T * (-(-n_heads // 16))
        pages = max(1, min(table.shape[1], -(-ctx.max_context // PAGE_TOKENS)))
        want = max(1, (4 * compute_units()) // max(1, n_tiles))          # blocks of one wave's work: a few a compute unit
        pps = max(1, -(-pages // min(pages, want, 16)))                  # (the merge kernel takes up to 16 parts)
        splits = -(-pages // pps)
        cu = None
        if splits > 1:
            floats = lib.llogos_latent_attn_workspace(T * n_heads, dv, splits)
            ws = _attn_workspace(q.device, floats)
    else:
        cu = ctx.cu_dev
        _need(cu is not None and cu.numel() == ctx.batch + 1, "latent attention: the step's token offsets are missing")
        n_tiles = sum(-(-(ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i]) * n_heads // 16) for i in range(ctx.batch))
    out = torch.empty((T, n_heads, dv), dtype=torch.bfloat16, device=q.device)
    code = lib.llogos_latent_attn_bf16(_p(out), dv, _p(q), _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(cu),
                                       _p(ctx.tok_pos), ctx.batch, T, n_heads, row, ctypes.c_float(scale), _p(head_sink),
                                       n_tiles, splits, pps, _p(ws), ctypes.c_longlong(ws.numel() if ws is not None else 0), _stream())
    if code == -2:
        return None
    _check(code, "latent_attention_mfma")
    return out


def head_products(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, w_kn: Optional[torch.Tensor] = None,
                  gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t, h, :N] = w[h] . a[t, h, :K] for every head h: a [T, H, >= K] and out [T, H, >= N] may be
    views with their own row and head strides; w [H, N, K] is dense.  w_kn [H, K, N]: the same matrices
    k-major, which steps of up to 16 rows stream instead (a kernel whose threads own an output each).
    gate float32 [T, >= H] (a view of wider rows will do): head h's outputs of row t are multiplied by
    sigmoid(gate[t, h])."""
    _need(a.is_cuda and w.is_cuda and out.is_cuda and w.is_contiguous(), "head_products: device tensors, dense w")
    _need(a.dim() == 3 and out.dim() == 3 and w.dim() == 3, "head_products: a [T, H, K], w [H, N, K], out [T, H, N]")
    T, H, K = a.shape
    N = w.shape[1]
    _need(w.shape == (H, N, K) and out.shape == (T, H, N), "head_products: shapes do not fit")
    _need(a.stride(2) == 1 and out.stride(2) == 1, "head_products: unit inner strides")
    gate_stride = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= H
              and gate.stride(1) == 1, "head_products: gate must be float32 [T, >= H]")
        gate_stride = gate.stride(0) if T > 1 else max(H, gate.stride(0))
    if w_kn is not None and 0 < T <= 16:
        _need(w_kn.is_cuda and w_kn.is_contiguous() and w_kn.shape == (H, K, N) and w_kn.dtype == w.dtype, "head_products: w_kn must be [H, K, N] like w")
        code = _lib().llogos_head_products_few(_p(out), _dt(out), out.stride(0), out.stride(1), _p(a), _dt(a), a.stride(0), a.stride(1),
                                               _p(w_kn), _dt(w_kn), T, H, N, K, _p(gate), gate_stride, _stream())
        if code != -2:
            _check(code, "head_products_few")
            return out
    if T:
        _check(_lib().llogos_head_products(_p(out), _dt(out), out.stride(0), out.stride(1), _p(a), _dt(a), a.stride(0), a.stride(1),
                                           _p(w), _dt(w), T, H, N, K, _p(gate), gate_stride, _stream()), "head_products")
    return out


def post_norm(x: torch.Tensor, delta: Optional[torch.Tensor], alpha: float, weight: torch.Tensor, eps: float,
              rows_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """The float32 stream x [T, H] becomes norm(alpha * x + delta) * weight in place (RMS norm, eps inside the
    root); `delta` is [T, H] or partial sums [parts, T, H], float32 or bfloat16, or None.  With `rows_dtype`
    the new rows are also returned in that type (for float32 that is x itself: nothing more is written)."""
    _dev(x, weight, delta)
    _need(x.dtype == torch.float32 and x.dim() == 2, "post_norm: x must be float32 [T, H]")
    T, H = x.shape
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "post_norm: weight must be float32 [H]")
    parts, part_stride = _parts(delta)
    if delta is not None:
        _need(tuple(delta.shape[-2:]) == (T, H), "post_norm: delta must have x's shape")
    rows = None
    if rows_dtype is not None and rows_dtype != torch.float32:
        rows = torch.empty((T, H), dtype=rows_dtype, device=x.device)
    if T:
        _check(_lib().llogos_post_norm(_p(x), _p(delta), _dt(delta) if delta is not None else F32, parts,
                                       ctypes.c_longlong(part_stride), ctypes.c_float(alpha), _p(weight), ctypes.c_float(eps), T, H,
                                       _p(rows), _DT[rows.dtype] if rows is not None else F32, _stream()), "post_norm")
    return x if (rows_dtype == torch.float32) else rows


RECURRENCE_SEGMENT = 0       # 0: chosen by the step; > 0 forces the segment length of the gated recurrence, -1 forbids segments (tests)


def recurrence_segments(lens: Sequence[int], channels: int, n_cus: Optional[int] = None) -> int:
    """The segment length for a step's gated recurrences (0: every sequence whole, one thread a channel).
    A whole sequence gives batch * channels threads, which run its tokens one after the other; segments
    run side by side at the price of a second pass over the inputs.  They pay when the sequences are
    long and their threads alone would leave most of the GPU idle."""
    if RECURRENCE_SEGMENT:
        return max(0, RECURRENCE_SEGMENT)
    longest = max(lens)
    if longest < 256:
        return 0
    n_cus = n_cus or compute_units()
    waves = len(lens) * ((channels + 63) // 64)
    if waves >= 8 * n_cus:
        return 0
    want = max(2, min(longest // 64, (8 * n_cus + waves - 1) // waves))
    return max(64, -(-longest // want))


def gated_recurrence(ctx, u: torch.Tensor, gates: torch.Tensor, block: int, r_bias: torch.Tensor, i_bias: torch.Tensor,
                     decay: torch.Tensor, y: torch.Tensor, state: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """S <- a S + sqrt(1 - a^2) * (i * u) with a = exp(-decay * r), r and i the sigmoids of the gate logits;
    returns S * gelu_tanh(y) as [T, C] in `out_dtype`.  u, y: float32 [T, C] (maybe columns of wider rows);
    gates float32 [T, >= 2 C] laid out in blocks of `block` channels as [r logits | i logits]; r_bias, i_bias,
    decay float32 [C]; state float32 [slots, C] (a view with its own slot stride will do): each sequence's S,
    read at the start of its tokens and written behind them."""
    for t_, name in ((u, "u"), (gates, "gates"), (y, "y")):
        _need(t_.is_cuda and t_.dtype == torch.float32 and t_.dim() == 2 and t_.stride(1) == 1, f"gated_recurrence: {name} must be float32 rows on the GPU")
    _dev(r_bias, i_bias, decay, ctx.slots, ctx.cu_dev)
    T, C = u.shape
    _need(T == ctx.n_tokens and y.shape == (T, C) and gates.shape[0] == T and gates.shape[1] >= 2 * C, "gated_recurrence: one row a token, 2 C gate logits")
    _need(block > 0 and C % block == 0, "gated_recurrence: the channels must divide into the blocks")
    for t_ in (r_bias, i_bias, decay):
        _need(t_.dtype == torch.float32 and t_.shape == (C,), "gated_recurrence: biases and decay must be float32 [C]")
    _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == C and state.stride(1) == 1,
          "gated_recurrence: state must be float32 [slots, C]")
    _need(ctx.cu_dev is not None or T == ctx.batch, "gated_recurrence: a step of several tokens a sequence needs the token offsets")
    ld = lambda t_, least: t_.stride(0) if T > 1 else max(least, t_.stride(0))
    out = torch.empty((T, C), dtype=out_dtype, device=u.device)
    seg_len, n_seg, seg_first, seg_a, seg_l = 0, 0, None, None, None
    if ctx.cu_dev is not None and not ctx.in_graph and RECURRENCE_SEGMENT >= 0:
        lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
        seg_len = recurrence_segments(lens, C)
        if seg_len > 0:
            first = [0]
            for n in lens:
                first.append(first[-1] + -(-n // seg_len))
            n_seg = first[-1]
            # the segments' offsets, made on the device from the step's token offsets (a copy from the host would
            # wait for the stream to drain), once a step for every layer that cuts it alike
            key = ("recurrence_segments", seg_len)
            seg_first = ctx.shared.get(key)
            if seg_first is None:
                counts = (ctx.cu_dev[1:] - ctx.cu_dev[:-1] + (seg_len - 1)) // seg_len
                seg_first = torch.zeros(ctx.batch + 1, dtype=torch.int32, device=u.device)
                seg_first[1:] = torch.cumsum(counts, 0)
                ctx.shared[key] = seg_first
            seg_a = torch.empty((n_seg, C), dtype=torch.float32, device=u.device)
            seg_l = torch.empty((n_seg, C), dtype=torch.float32, device=u.device)
    slot_stride = state.stride(0) if state.shape[0] > 1 else max(C, state.stride(0))
    _check(_lib().llogos_gated_recurrence(
        _p(out), _DT[out_dtype], _p(u), ld(u, C), _p(gates), ld(gates, 2 * C), int(block), _p(r_bias), _p(i_bias), _p(decay),
        _p(y), ld(y, C), _p(state), ctypes.c_longlong(slot_stride), _p(ctx.slots), _p(ctx.cu_dev), T, ctx.batch, C,
        int(seg_len), int(n_seg), _p(seg_first), _p(seg_a), _p(seg_l), _stream()), "gated_recurrence")
    return out


def rotary_prepare(ctx, qkv: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype, n_heads: int, n_kv_heads: int,
                   dim: int, v_dim: int, maps: int, rot: int, pairing: int, cs: Optional[torch.Tensor],
                   q_norm_w: Optional[torch.Tensor], k_norm_w: Optional[torch.Tensor], unit_after: bool, eps: float,
                   k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor], table: Optional[torch.Tensor],
                   writes: bool = True) -> torch.Tensor:
    """From projected rows [q | k | v] ([T, >= W] or partial sums [parts, T, >= W], float32 or the cache's type,
    plus `bias` [W]; W = (n_heads + n_kv_heads) * maps * dim + n_kv_heads * v_dim): every run of `dim` values of q
    and k (a head, or one of a head's `maps` score maps) gets an RMS norm with a shared weight where one is given,
    then the rotation of its first `rot` dimensions by the table `cs` [T, rot / 2, 2], then, with `unit_after`,
    is divided by its root mean square.  q comes back [T, n_heads * maps * dim] in `out_dtype`; a kv head's `maps`
    key runs go side by side into its key page row, its v_dim values into its value page row.  writes False:
    only q is made."""
    _need(qkv.is_cuda and qkv.stride(-1) == 1 and (qkv.dtype == torch.float32 or qkv.dtype == out_dtype),
          "rotary_prepare: rows must be float32 or the cache's type, on the GPU")
    _dev(bias, q_norm_w, k_norm_w, cs, table, ctx.tok_seq, ctx.tok_pos)
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    Wq, Wk, Wv = n_heads * maps * dim, n_kv_heads * maps * dim, n_kv_heads * v_dim
    width = Wq + ((Wk + Wv) if writes else 0)
    _need(qkv.shape[-1] >= width and T == ctx.n_tokens, f"rotary_prepare: rows of at least {width} values, one a token")
    _need(maps >= 1 and 0 < dim <= GENERIC_MAX_HEAD_DIM and 0 < v_dim <= GENERIC_MAX_HEAD_DIM, "rotary_prepare: head sizes out of range")
    _need(rot % 2 == 0 and 0 <= rot <= dim and pairing in (0, 1), "rotary_prepare: the rotated width must be even and within a run")
    if rot:
        _need(cs is not None and cs.dtype == torch.float32 and tuple(cs.shape) == (T, rot // 2, 2), "rotary_prepare: rotary table shape")
    row_stride = qkv.stride(-2) if T > 1 else max(Wq + Wk + Wv, qkv.stride(-2))
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() >= width, f"rotary_prepare: bias must be float32 [{width}]")
    for wgt in (q_norm_w, k_norm_w):
        if wgt is not None:
            _need(wgt.dtype == torch.float32 and wgt.shape == (dim,), "rotary_prepare: a norm weight must be float32 [dim]")
    kd = vd = 0
    if writes:
        _need(k_pool is not None and v_pool is not None and table is not None, "rotary_prepare: cache missing")
        _i32(table, "table")
        _need(k_pool.dtype == out_dtype and v_pool.dtype == out_dtype, "rotary_prepare: cache type differs")
        kd, vd = _page_dims(k_pool, v_pool, n_kv_heads, "rotary_prepare")
        _need(kd >= maps * dim and vd >= v_dim and table.dim() == 2, "rotary_prepare: pages narrower than the heads")
    q_out = torch.empty((T, Wq), dtype=out_dtype, device=qkv.device)
    _check(_lib().llogos_rotary_prepare(
        _p(qkv), _dt(qkv), parts, ctypes.c_longlong(part_stride), row_stride, _p(bias), _p(q_out), _DT[out_dtype], n_heads * maps,
        n_kv_heads if writes else 0, dim, v_dim, maps, rot, pairing, _p(q_norm_w), _p(k_norm_w), 1 if unit_after else 0,
        ctypes.c_float(eps), _p(cs), _p(k_pool) if writes else None, _p(v_pool) if writes else None, kd, vd,
        _p(table) if writes else None, table.stride(0) if (writes and table is not None) else 0, _p(ctx.tok_seq), _p(ctx.tok_pos),
        T, _stream()), "rotary_prepare")
    return q_out


DIFF_MFMA = True             # False keeps differential attention off the matrix cores (tests)
DIFF_PREFILL_HALVES = 0      # 0: chosen by the step; 1 or 2 forces the sets of waves a block of its prompt kernel (tests)


def diff_attention(ctx, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, table: torch.Tensor, n_heads: int,
                   n_kv_heads: int, dim: int, v_dim: int, scale: float, lam: float, out_scale: float, eps: float,
                   window: int = 0, sinks: int = 0) -> torch.Tensor:
    """Differential attention of the step's query rows q [T, n_heads * 2 * dim] (head by head [map 1 | map 2]) over
    their sequences' pages, whose key rows hold both maps' keys side by side: two softmax maps over the same
    values, out = (a_1 - lam * a_2) / rms(a_1 - lam * a_2) * out_scale per head.  Returns [T, n_heads * v_dim]."""
    T = ctx.n_tokens
    _dev(q, k_pool, v_pool, table, ctx.tok_seq, ctx.tok_pos)
    _i32(table, "table")
    _need(q.dtype == k_pool.dtype and tuple(q.shape) == (T, n_heads * 2 * dim), "diff_attention: q must be [T, heads * 2 * dim] of the cache's type")
    _need(n_heads % n_kv_heads == 0, "diff_attention: heads must be a multiple of kv heads")
    kd, vd = _page_dims(k_pool, v_pool, n_kv_heads, "diff_attention")
    _need(v_pool is not None and kd >= 2 * dim and vd >= v_dim, "diff_attention: pages narrower than the heads")
    _need(2 * dim <= GENERIC_MAX_HEAD_DIM and 0 < v_dim <= GENERIC_MAX_HEAD_DIM, "diff_attention: head sizes out of range")
    out = torch.empty((T, n_heads * v_dim), dtype=q.dtype, device=q.device)
    if q.dtype == torch.bfloat16 and DIFF_MFMA and q.is_contiguous() and kd == 2 * dim and vd == v_dim:
        # head shapes the matrix-core kernels take run there; -2 says that this one is none of them
        lib = _lib()
        if ctx.is_decode:
            width = table.shape[1]
            _need(table.shape[0] == T and ctx.tok_pos.numel() == T, "diff_attention: one table row and position a sequence")
            ws = _attn_workspace(q.device, lib.llogos_diff_attn_decode_workspace(T, n_heads, n_kv_heads, v_dim, width))
            code = lib.llogos_diff_attn_decode_bf16(
                _p(out), _p(q), q.stride(0), _p(k_pool), _p(v_pool), _p(table), table.stride(0), width, _p(ctx.tok_pos), T,
                n_heads, n_kv_heads, dim, v_dim, ctypes.c_float(scale), int(window), int(sinks), ctypes.c_float(lam),
                ctypes.c_float(out_scale), ctypes.c_float(eps), _p(ws), ctypes.c_longlong(ws.numel()), _stream())
        else:
            cu = ctx.cu_dev
            _need(cu is not None and cu.numel() == ctx.batch + 1, "diff_attention: the step's token offsets are missing")
            lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
            n_tiles = sum(-(-n // 128) for n in lens)
            halves = DIFF_PREFILL_HALVES or prefill_halves(lens, getattr(ctx, "starts", None), 2 * n_heads)
            ws = torch.empty(lib.llogos_diff_attn_prefill_workspace(T, n_heads, v_dim), dtype=torch.float32, device=q.device)
            code = lib.llogos_diff_attn_prefill_bf16(
                _p(out), _p(q), q.stride(0), _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(cu), _p(ctx.tok_pos),
                ctx.batch, T, n_tiles, n_heads, n_kv_heads, dim, v_dim, ctypes.c_float(scale), int(window), int(sinks),
                ctypes.c_float(lam), ctypes.c_float(out_scale), ctypes.c_float(eps), int(halves), _p(ws),
                ctypes.c_longlong(ws.numel()), _stream())
        if code != -2:
            _check(code, "diff_attention")
            return out
    _check(_lib().llogos_diff_attention_generic(
        _p(out), _p(q), _dt(q), q.stride(0), _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(ctx.tok_seq), _p(ctx.tok_pos),
        T, n_heads, n_kv_heads, dim, v_dim, kd, vd, ctypes.c_float(scale), int(window), int(sinks), ctypes.c_float(lam),
        ctypes.c_float(out_scale), ctypes.c_float(eps), _stream()), "diff_attention_generic")
    return out


# ----------------------------------------------------------------------------
# dispatch: which kernel serves a call
# ----------------------------------------------------------------------------
_compute_units = {}


def compute_units(device=None) -> int:
    """Compute units of the GPU the products are planned for, read from the device once (256 on
    an MI355X; that number also stands in where no GPU is visible, for planning on the host)."""
    if not torch.cuda.is_available():
        return 256
    index = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    if index not in _compute_units:
        _compute_units[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return _compute_units[index]


SKINNY_MAX_ROWS = 64
LDS_MAX_ROWS = 128          # rows the LDS few-row product takes without a fused producer


def lds_splits(M: int, N: int, K: int, n_cus: Optional[int] = None) -> int:
    """Blocks along k for the LDS few-row product.  Measured on the MI355X, three things decide:
    how evenly the blocks fill the compute units (544 blocks on 256 units run as long as 768),
    whether there are enough of them to keep the memory system busy (about 1.5 a unit), and the
    float32 partial sums every further block along k writes and the consumer reads (they cost
    about 6 M / K of the weights' time each).  64 and more rows of activations leave LDS for two
    blocks a unit, so blocks come in rounds of twice the units there.  More blocks along k are taken only
    for a clear gain (8 %), since they also cost the consumer a fused form or a launch."""
    n_cus = n_cus or compute_units()
    n_blocks = -(-N // 64)
    chunks = -(-K // 256)
    rows = 16 if M <= 16 else (32 if M <= 32 else (64 if M <= 64 else 128))
    per_round = n_cus * (2 if rows >= 64 else 1)
    best, best_score, seen = 1, -1.0, set()
    for s in range(1, 9):
        per = -(-chunks // s)
        parts = -(-chunks // per)
        if parts in seen or (parts > 1 and per < 2):
            continue
        seen.add(parts)
        blocks = n_blocks * parts
        evenness = blocks / (-(-blocks // per_round) * per_round)
        enough = min(1.0, blocks / (1.5 * n_cus))
        partial_sums = 1.0 + (parts - 1) * 6.0 * rows / K
        score = evenness * enough / partial_sums * (1.0 - 0.01 * (parts - 1))
        if score > best_score * 1.08:
            best, best_score = parts, score
    return best


def stationary_strips(N: int, K: int, n_cus: Optional[int] = None) -> int:
    """Strips of 16 rows of w a block of the activation-stationary product streams.  More strips
    spread the activations' loads over more weights; the blocks must still fill the compute
    units evenly (598 blocks on 256 units were measured at 3.9 TB/s where 448 reach 5.5) and
    leave about seven waves a unit."""
    n_cus = n_cus or compute_units()
    waves = 4 if K <= 4096 else 8
    n_strips = -(-N // 16)
    best, best_score = 2, -1.0
    for strips in range(2, 17):
        blocks = -(-n_strips // strips)
        evenness = blocks / (-(-blocks // n_cus) * n_cus)
        enough = min(1.0, blocks * waves / (7.0 * n_cus))
        score = evenness * enough / (1.0 + 0.4 / strips)
        if score >= best_score:
            best, best_score = strips, score
    return best


def resident_strips(M: int, N: int, K: int, n_cus: Optional[int] = None) -> Optional[Tuple[int, int]]:
    """(parts of k, strips per block) for the few-row product whose operands go straight into
    LDS, or None where it is not the faster one.  It pays for 17 to 64 rows on a tall, large
    matrix when its blocks, 5 to 9 strips high, are all resident at once (two to a compute
    unit) and fill most of those places, while the LDS few-row product's 64-row blocks either
    need a second round or leave a fifth more of the places empty: then the activations are
    read once per 80 to 144 rows of w and nothing waits for a second round (measured on the
    gate/up matrices of eight model sizes: 6 to 20 % faster where this says so, level or
    slower where it does not, among them everything below 24576 rows)."""
    if not (16 < M <= 64 and N >= 24576 and K % 64 == 0):
        return None
    n_cus = n_cus or compute_units()
    places = 2 * n_cus
    other = -(-N // 64) * lds_splits(M, N, K, n_cus)
    other_fill = other / places if other <= places else 0.0
    n_strips = -(-N // 16)
    best, best_fill = None, 0.0
    for strips in (9, 8, 7, 6, 5):
        for parts in (1, 2):
            if parts > 1 and K < 512 * parts:
                continue
            blocks = -(-n_strips // strips) * parts
            if blocks <= places and blocks / places > best_fill:
                best, best_fill = (parts, strips), blocks / places
    if best is None or best_fill < 0.75 or best_fill - other_fill < 0.2:
        return None
    return best


def skinny_plan(M: int, N: int, K: int) -> Tuple[str, int, int]:
    """(kernel, blocks along k, 16-row blocks of w per wave) for the few-row product.
    'strips': both operands straight into LDS, blocks of several strips (see resident_strips).
    'stationary': activations held in registers while strips of w stream past; best for few
    rows and very many rows of w (gate/up, the head).  'regs': every wave fetches its own
    activation fragments; for up to 4 rows where k is too long for 'stationary'.  'lds': the
    block shares the activations through LDS; its speed hardly depends on the number of rows.
    The plan depends on the shape and on the number of rows rounded up to 16, 32 or 64, so a
    row's additions come in the same order for every batch of that class."""
    if N >= 16384 and K <= 4096 and (M <= 8 or (M <= 16 and N >= 65536)):
        return "stationary", 1, stationary_strips(N, K)       # third value: strips per block
    if N >= 16384 and 4096 < K <= 8192 and M <= 16:           # 8 waves a block
        return "stationary", 1, stationary_strips(N, K)
    if M <= 4 and N >= 16384:
        strips = -(-N // 16)
        return "regs", max(1, min(-(-1024 // strips), K // 1024, 8)), 1
    resident = resident_strips(M, N, K)
    if resident is not None:
        return "strips", resident[0], resident[1]             # third value: strips per block
    return "lds", lds_splits(M, N, K), 1


def long_inner(w: torch.Tensor) -> bool:
    """Whether w [N, K] has few rows for its length (a feed-forward's down projection).  For 65
    to 128 rows of activations the library's product leaves most compute units idle on such a
    matrix (75 us measured for [4096, 14336] at 128 rows, 1.6 TB/s), and the LDS few-row
    product with blocks along k is faster (44 us); on the other layer shapes the library is."""
    return w.dtype == torch.bfloat16 and w.shape[1] >= 2 * w.shape[0]


def gemm_skinny_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int = 1, row_blocks: int = 1) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product on the matrix cores: [parts, M, N], where parts > 1 are
    float32 partial sums over ranges of k that the consumer adds (then no bias is applied
    here).  None when the shape is not one the kernel takes."""
    M, K = a.shape
    N = w.shape[0]
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0
            and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_skinny_bf16(
        _p(out), _DT[out_dtype], _p(a), _p(w), _p(bias), M, N, K, a.stride(0), N,
        ctypes.c_longlong(M * N), int(splits), int(row_blocks), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_bf16")
    return out


def gemm_skinny_stationary_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor],
                                out_dtype: torch.dtype, strips: int = 4) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product with the activations held in registers while `strips` strips
    of 16 rows of w stream past: up to 16 rows, K <= 8192.  [1, M, N]; None for other shapes."""
    if a.dim() != 2:
        return None
    M, K = a.shape
    N = w.shape[0]
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < M <= 16 and K <= 8192 and K % 8 == 0
            and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    out = torch.empty((1, M, N), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_skinny_stationary_bf16(
        _p(out), _DT[out_dtype], _p(a), _p(w), _p(bias), M, N, K, a.stride(0), N, int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_stationary_bf16")
    return out


def gemm_skinny_lds_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                         splits: int = 1, row_blocks: int = 1, swiglu: bool = False) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product with the activations shared through LDS: [parts, M, N].
    With `swiglu`, `a` is the fused gate/up product ([M, 2 K] bfloat16 or float32 partial sums
    [parts, M, 2 K]) and silu(gate) * up is made on the way.  None for shapes it does not take."""
    if swiglu:
        a_parts, a_stride = _parts(a)
        M, K2 = a.shape[-2:]
        K = K2 // 2
        if a.dtype == torch.float32:
            mode = 1
        elif a.dtype == torch.bfloat16 and a_parts == 1:
            mode = 2
        else:
            return None
        lda = a.stride(-2)
    else:
        if a.dtype != torch.bfloat16 or a.dim() != 2:
            return None
        a_parts, a_stride, mode = 1, 0, 0
        M, K = a.shape
        lda = a.stride(0)
    N = w.shape[0]
    if not (w.dtype == torch.bfloat16 and 0 < M <= (SKINNY_MAX_ROWS if swiglu else LDS_MAX_ROWS) and K % 8 == 0
            and a.stride(-1) == 1 and lda % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.is_contiguous()
            and a_stride % 4 == 0):
        return None
    _dev(w, bias)
    _need(w.dim() == 2 and w.shape[1] == K, f"gemm: w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_lds_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_skinny_lds_bf16(
        _p(out), _DT[out_dtype], _p(a), mode, lda, a_parts, ctypes.c_longlong(a_stride), _p(w), _p(bias),
        M, N, K, N, ctypes.c_longlong(M * N), int(splits), int(row_blocks), _stream())
    if code == -2:
        return None
    _check(code, "gemm_skinny_lds_bf16")
    return out


def gemm_strips_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int, strips: int) -> Optional[torch.Tensor]:
    """The bfloat16 product for up to 128 rows whose operands go straight into LDS, several
    stages ahead, with blocks of `strips` 16-row strips of w: [parts, M, N], the same parts of k
    and the same sums as gemm_skinny_lds_bf16.  None for shapes it does not take."""
    if a.dtype != torch.bfloat16 or a.dim() != 2 or w.dtype != torch.bfloat16 or w.dim() != 2:
        return None
    M, K = a.shape
    N = w.shape[0]
    if not (0 < M <= LDS_MAX_ROWS and K % 64 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and w.shape[1] == K
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.is_contiguous() and 2 <= strips <= 9):
        return None
    _dev(w, bias)
    _need(a.is_cuda and a.device == w.device, "gemm: a and w must be on the same GPU")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_skinny_lds_parts(K, int(splits))
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_strips_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(w), _p(bias), M, N, K, N,
                                       ctypes.c_longlong(M * N), int(splits), int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_strips_bf16")
    return out


class PackedWeight:
    """A bfloat16 matrix [N, K] in the order in which the matrix cores take it (pack_weights): blocks of
    64 rows, steps of 32 values of k, one 16-byte fragment a lane, zero-padded.  The few-row
    products stream it as one contiguous run per block."""
    __slots__ = ("data", "N", "K", "gate_rows")

    def __init__(self, data: torch.Tensor, N: int, K: int, gate_rows: int = 0):
        # gate_rows > 0: w is [gate; up] of gate_rows rows each and the packed strips of 16 rows alternate
        # between the two, for the product that makes silu(gate) * up in its epilogue (and for no other)
        self.data, self.N, self.K, self.gate_rows = data, N, K, gate_rows

    def rows(self, n: int) -> Optional["PackedWeight"]:
        """The first n rows as a packed matrix of their own (whole blocks of 64 rows only)."""
        if n == self.N:
            return self
        if n <= 0 or n > self.N or n % 64 or self.gate_rows:
            return None
        per_block = -(-self.K // 32) * 2048                  # bfloat16 elements of one block of rows
        return PackedWeight(self.data[: (n // 64) * per_block], n, self.K)


def packed_weight_bytes(N: int, K: int) -> int:
    return -(-N // 64) * -(-K // 32) * 4096


def pack_weights(w: torch.Tensor, gate_rows: int = 0) -> PackedWeight:
    """A packed copy of the bfloat16 matrix w [N, K].  gate_rows: w is a gate matrix on top of an up
    matrix of gate_rows rows each (a multiple of 16), and strips of 16 gate rows and of the 16 up
    rows of the same columns follow one another in the copy (see gemm_packed_gated_bf16)."""
    _dev(w)
    _need(w.dtype == torch.bfloat16 and w.dim() == 2, "pack_weights: w must be bfloat16 [N, K]")
    N, K = w.shape
    _need(gate_rows == 0 or (gate_rows % 16 == 0 and N == 2 * gate_rows), "pack_weights: gate and up of a multiple of 16 rows each")
    data = torch.empty(packed_weight_bytes(N, K) // 2, dtype=torch.bfloat16, device=w.device)
    _check(_lib().llogos_pack_weights(_p(data), _p(w), N, K, int(gate_rows), _stream()), "pack_weights")
    return PackedWeight(data, N, K, int(gate_rows))


def gemm_packed_gated_bf16(a: torch.Tensor, pw: PackedWeight, out_dtype: torch.dtype, chunk: int = 256) -> Optional[torch.Tensor]:
    """silu(a . gate^T) * (a . up^T) as [M, gate_rows] for up to 64 rows of bfloat16 activations, on a matrix
    packed with gate_rows: the gate/up product stays in registers.  None for shapes it does not take."""
    if pw.gate_rows <= 0 or a.dtype != torch.bfloat16 or a.dim() != 2:
        return None
    M, K = a.shape
    if not (K == pw.K and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(pw.data)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    out = torch.empty((M, pw.gate_rows), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_packed_gated_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(pw.data), M, pw.N, K,
                                                pw.gate_rows, int(chunk), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_gated_bf16")
    return out


def packed_plan(M: int, N: int, K: int) -> Tuple[int, int]:
    """(blocks along k, values of k per LDS buffer) for the few-row product on packed weights: the
    blocks along k as for the row-major form (the same trade of evenness, enough blocks and the
    cost of partial sums, measured again on packed weights), and the shorter buffer for up to 16
    rows, where it was 2 to 5 % faster.  One plan per class of row count (16, 32, 64); the kernel itself
    works in tiles of 16 rows, 1 to 4 of them (33 to 48 rows take three: 41.7 us against 46.1 for the 8B
    gate/up matrix), which changes no sum."""
    return lds_splits(M, N, K), (128 if M <= 16 else 256)


def gemm_packed_bf16(a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                     splits: int = 1, chunk: int = 256, swiglu: bool = False) -> Optional[torch.Tensor]:
    """The few-row bfloat16 product on packed weights: [parts, M, N]; parts > 1 are float32 partial
    sums over ranges of k that the consumer adds.  With `swiglu`, `a` is the fused gate/up product
    ([M, 2 K] bfloat16 or float32 partial sums [parts, M, 2 K]) and silu(gate) * up is made on the
    way.  None for shapes it does not take."""
    if swiglu:
        a_parts, a_stride = _parts(a)
        M, K2 = a.shape[-2:]
        K = K2 // 2
        if a.dtype == torch.float32:
            mode = 1
        elif a.dtype == torch.bfloat16 and a_parts == 1:
            mode = 2
        else:
            return None
        lda = a.stride(-2)
    else:
        if a.dtype != torch.bfloat16 or a.dim() != 2:
            return None
        a_parts, a_stride, mode = 1, 0, 0
        M, K = a.shape
        lda = a.stride(0)
    N = pw.N
    if not (K == pw.K and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 and a.stride(-1) == 1 and lda % 8 == 0
            and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0 and a_stride % 4 == 0):
        return None
    _dev(pw.data, bias)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    lib = _lib()
    parts = lib.llogos_gemm_packed_parts(K, int(splits), int(chunk))
    _need(parts >= 1, "gemm: the LDS buffer holds 128 or 256 values of k")
    if parts > 1:
        _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
        out_dtype = torch.float32
    out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_packed_bf16(
        _p(out), _DT[out_dtype], _p(a), mode, lda, a_parts, ctypes.c_longlong(a_stride), _p(pw.data), _p(bias),
        M, N, K, N, ctypes.c_longlong(M * N), int(splits), int(chunk), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_bf16")
    return out


RESIDUAL_MAX_ROWS = 16     # rows at most of the product that adds itself to the residual stream
# "on" (the default): steps of up to 16 rows close a mixer and a feed-forward with gemm_residual_bf16 and
# open the next with gemm_packed_unscaled_bf16 where the shapes allow; "off": the products in parts and
# the norm's own kernel everywhere.  LLOGOS_RESIDUAL_PRODUCT in the environment sets the default.
RESIDUAL_PRODUCT = os.environ.get("LLOGOS_RESIDUAL_PRODUCT", "on")


@dataclass
class RowSquares:
    """What a product that has added itself to the residual stream x leaves beside it: sums [blocks, 16],
    float32, each of the product's blocks holding for each row of x the sum of the squares of its 16 or 32
    columns.  A norm over the rows of x needs no other pass over them (gemm_packed_unscaled_bf16)."""
    sums: Optional[torch.Tensor]                # None: the product left nothing but the complete stream
    width: int                                  # columns of x that the sums cover
    unscaled: Optional[torch.Tensor] = None     # bfloat16 [M, width]: x * norm_w, the rmsnorm's rows without their scale
    norm_w: Optional[torch.Tensor] = None       # the weight that `unscaled` was made with


def residual_plan(M: int, N: int, K: int, n_cus: Optional[int] = None) -> Tuple[int, int]:
    """(waves of a block, strips of 16 rows of w a block) of gemm_residual_bf16; (0, 0): not served (then the
    product in parts over k and the norm's own kernel do the work).  A block owns its rows of w and all of k,
    and a compute unit streams what its blocks own at a bounded rate: the blocks have to fill the units evenly,
    one block a unit at best.  Measured on the MI355X (256 units) at 1, 8 and 16 rows against the product in
    parts plus the norm kernel (us):
      N / 16 <= units (1B, 3B, 8B widths): blocks of one strip, 8 waves: 8B o 9.0 against 12.4, down 21.0
        against 24.2 (two strips a block: 10.5 and 27.8: half the units idle);
      more strips than units: two strips a block, which share a wave's copy of the activations: 70B (256
        blocks) o 24.2 against 27.5, down 71.2 against 79.4 (one strip a block, two blocks a unit: 76.1); 14B
        (160 blocks) o 12.8 against 16.1; its down projection, 89 M weights on 160 of 256 units, only up to 4
        rows (31.6 against 35.4 at one row, 34.6 against 33.6 at 8, 38.4 against 34.1 at 16)."""
    if RESIDUAL_PRODUCT != "on" or not (0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0):
        return 0, 0
    n_cus = n_cus or compute_units()
    strips = -(-N // 16)
    waves = 8 if K >= 1024 else 4
    if N * K <= (1 << 22):                    # so small that only the number of kernels counts
        return waves, 1
    if strips <= n_cus:
        return (waves, 1) if strips >= n_cus // 2 else (0, 0)
    blocks = -(-strips // 2)
    if blocks < (3 * n_cus) // 4 and N * K > (1 << 25) and M > 4:
        return 0, 0
    return 8, 2


def gemm_residual_bf16(x: torch.Tensor, a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor],
                       waves: int, norm_w: Optional[torch.Tensor] = None, strips: int = 1) -> Optional[RowSquares]:
    """x [M, N] (float32, in place) += a [M, K] . w^T (+ bias) for up to 16 rows of bfloat16 activations in
    one kernel, every sum in an order fixed by the shapes; returns the sums of squares of x's new rows, by
    strips of 16 columns, and with `norm_w` [N] also x * norm_w in bfloat16 (the rows of the rmsnorm with
    that weight, without their scale).  None for shapes it does not take."""
    if a.dtype != torch.bfloat16 or a.dim() != 2 or x.dim() != 2 or x.dtype != torch.float32 or pw.gate_rows:
        return None
    M, K = a.shape
    N = pw.N
    if not (K == pw.K and x.shape == (M, N) and 0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1
            and a.stride(0) % 8 == 0 and x.stride(1) == 1 and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(x, a, pw.data, bias, norm_w)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
    unscaled = None
    if norm_w is not None:
        _need(norm_w.dtype == torch.float32 and norm_w.shape == (N,) and norm_w.is_contiguous(), "gemm: norm weight must be float32 [N]")
        unscaled = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    sums = torch.empty((-(-(-(-N // 16)) // int(strips)), 16), dtype=torch.float32, device=x.device)
    code = _lib().llogos_gemm_residual_bf16(_p(x), x.stride(0), _p(sums), _p(unscaled), N, _p(norm_w), _p(a), a.stride(0),
                                            _p(pw.data), _p(bias), M, N, K, int(waves), int(strips), _stream())
    if code == -2:
        return None
    _check(code, "gemm_residual_bf16")
    return RowSquares(sums, N, unscaled, norm_w)


def gemm_packed_unscaled_bf16(squares: RowSquares, eps: float, pw: PackedWeight, bias: Optional[torch.Tensor],
                              out_dtype: torch.dtype, splits: int = 1, chunk: int = 128) -> Optional[torch.Tensor]:
    """The few-row product on packed weights with an rmsnorm's rows as its activations, of which `squares`
    holds x * norm_w in bfloat16 and the sums of squares of x (gemm_residual_bf16 with norm_w): the rows'
    scale 1 / sqrt(mean square + eps) is applied to the product, in float32.  On a matrix packed with
    gate_rows the result is silu(gate) * up [M, gate_rows], otherwise [parts, M, N] as gemm_packed_bf16 (a
    bias is added after the scale).  None for shapes it does not take."""
    a = squares.unscaled
    if a is None:
        return None
    M, K = a.shape
    N = pw.N
    if not (K == pw.K and squares.width == K and 0 < M <= RESIDUAL_MAX_ROWS and K % 8 == 0 and a.stride(1) == 1
            and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0 and pw.data.data_ptr() % 16 == 0):
        return None
    _dev(a, squares.sums, pw.data, bias)
    _need(squares.sums.dtype == torch.float32 and squares.sums.dim() == 2 and squares.sums.shape[1] == RESIDUAL_MAX_ROWS
          and squares.sums.is_contiguous() and squares.sums.shape[0] >= 1 and a.dtype == torch.bfloat16,
          "gemm: the sums of squares are float32 [parts, 16], the unscaled rows bfloat16")
    lib = _lib()
    gated = pw.gate_rows > 0
    if gated:
        if bias is not None:
            return None
        parts, cols = 1, pw.gate_rows
        out = torch.empty((M, cols), dtype=out_dtype, device=a.device)
    else:
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.shape == (N,), "gemm: bias must be float32 [N]")
        parts = lib.llogos_gemm_packed_parts(K, int(splits), int(chunk))
        _need(parts >= 1, "gemm: the LDS buffer holds 128 or 256 values of k")
        if parts > 1:
            _need(bias is None, "gemm: a product in parts leaves the bias to its consumer")
            out_dtype = torch.float32
        cols = N
        out = torch.empty((parts, M, N), dtype=out_dtype, device=a.device)
    code = lib.llogos_gemm_packed_unscaled_bf16(
        _p(out), _DT[out_dtype], _p(a), a.stride(0), _p(squares.sums), squares.sums.shape[0], K,
        ctypes.c_float(eps), _p(pw.data), _p(bias), M, N, K, cols, ctypes.c_longlong(M * N), int(splits), int(chunk),
        int(gated), _stream())
    if code == -2:
        return None
    _check(code, "gemm_packed_unscaled_bf16")
    return out


# Which product serves many rows of bfloat16 (prompts): "auto" (the default): the hand-written tiled
# product (gemm_tiles_bf16 on the packed copy) where it was measured faster than the library's, which is
# the gate/up product with its SwiGLU epilogue from TILES_MIN_ROWS rows on, and the library's product
# elsewhere (as the reference uses a library there); "tiles": the hand-written one wherever it applies;
# "library": the library's everywhere.  LLOGOS_PROMPT_PRODUCT in the environment sets the default.
PROMPT_PRODUCT = os.environ.get("LLOGOS_PROMPT_PRODUCT", "auto")
TILES_MIN_ROWS, TILES_MAX_ROWS, TILES_MAX_K = 1024, 2048, 5120


def tiles_serve_gated(M: int, K: int = 0) -> bool:
    """Whether the tiled product makes silu(gate) * up for M rows of K values (rather than the library's product
    and a SwiGLU pass): by default from TILES_MIN_ROWS to TILES_MAX_ROWS rows with k up to TILES_MAX_K, where
    it was measured level or ahead (tiled against library + SwiGLU, us, sustained: 1B 63 / 67 at 1,024 rows,
    119 / 120 at 2,048; 8B 225 / 217 and 405 / 391, level inside the model; 14B 343 / 413 and 614 / 630).
    The library gains with the rows and with k (8B: 1.11 PFLOP/s at 1,024 rows, 1.34 from 4,096 on; 70B 1.41
    to 1.47) where the tiled product stays at 1.2: 8B at 4,096 rows 825 / 727, 70B at 2,048 rows 1,516 / 1,363,
    a 16,384-token prompt of the 8B sizes 278 ms against 268."""
    if PROMPT_PRODUCT == "tiles":
        return True
    return PROMPT_PRODUCT == "auto" and TILES_MIN_ROWS <= M <= TILES_MAX_ROWS and K <= TILES_MAX_K


def tiles_plan(M: int, N: int, K: int) -> Optional[Tuple[int, int]]:
    """(parts of k, token_tiles) with which the tiled product serves a plain product of M rows, or None where
    the library's does.  Measured on the MI355X at the layer sizes of 8B, 14B and 70B models: a matrix that
    is much longer than high (a feed-forward's down projection) with 129 to 1,024 rows of activations is where
    the library is furthest from its best (14B, 256 rows: 119 us against 65; 70B: 291 against 143; 8B, 512 rows:
    88 against 68), and blocks along k fill the compute units that its few row tiles leave idle.  Elsewhere
    the library's product was level or ahead (by 10 to 25 % from 2,048 rows on)."""
    if PROMPT_PRODUCT == "library" or M <= SKINNY_MAX_ROWS or K % 64:
        return None
    if PROMPT_PRODUCT == "tiles":
        return 1, 0
    if K >= 2 * N and LDS_MAX_ROWS < M <= 1024:
        parts, token_tiles = (4, 2) if M <= 256 else ((4, 0) if M <= 512 else (2, 0))
        while parts > 1 and (K // 64) // parts < 2:
            parts //= 2
        return parts, token_tiles
    return None


def gemm_tiles_bf16(a: torch.Tensor, pw: PackedWeight, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
                    parts: int = 1, token_tiles: int = 0) -> Optional[torch.Tensor]:
    """a [M, K] . w^T on the packed copy of w for any number of rows (tiles of 256 or 128 tokens x 256 rows,
    v_mfma_f32_32x32x16_bf16): [M, N] with the bias added, or, for a matrix packed with gate_rows,
    [M, gate_rows] = silu(gate) * up; with parts > 1 float32 partial sums [parts, M, N] over ranges of k.
    token_tiles: 4 or 2 force tiles of 256 or 128 tokens, 0 lets the launch choose.
    None for shapes it does not take (K no multiple of 64, parts of fewer than 128 values of k)."""
    if a.dtype != torch.bfloat16 or a.dim() != 2:
        return None
    M, K = a.shape
    if not (K == pw.K and M > 0 and K % 64 == 0 and a.stride(1) == 1 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0):
        return None
    gated = pw.gate_rows > 0
    _dev(pw.data, bias)
    _need(a.is_cuda and a.device == pw.data.device, "gemm: a and w must be on the same GPU")
    _need(not (gated and bias is not None), "gemm: the gated product takes no bias")
    _need(parts >= 1 and not (gated and parts > 1), "gemm: the gated product comes in one part")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (pw.N,), "gemm: bias must be float32 [N]")
        _need(parts == 1, "gemm: a product in parts leaves the bias to its consumer")
    if parts > 1:
        out_dtype = torch.float32
    width = pw.gate_rows if gated else pw.N
    out = torch.empty((parts, M, width), dtype=out_dtype, device=a.device)
    code = _lib().llogos_gemm_tiles_bf16(_p(out), _DT[out_dtype], _p(a), a.stride(0), _p(pw.data), _p(bias), M, pw.N, K,
                                         width, ctypes.c_longlong(M * width), int(gated), int(parts), int(token_tiles),
                                         compute_units(a.device), _stream())
    if code == -2:
        return None
    _check(code, "gemm_tiles_bf16")
    return out[0] if parts == 1 else out


def gemm_product(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, swiglu_input: bool = False,
                 f32_ok: bool = False, packed: Optional[PackedWeight] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T without bias, as [M, N] of `out_dtype` or as float32 partial sums
    [parts, M, N] for a consumer that adds them (rmsnorm, qk_rope_cache, swiglu, sum_parts).
    With `swiglu_input`, `a` is a fused gate/up product ([M, 2 K] or parts of it) and the
    product is taken of silu(gate) * up.  With `f32_ok` the consumer also takes one float32
    [M, N], which spares the result a rounding to bfloat16.

    float32 operands: plain FMAs in 32-bit throughout.  bfloat16 operands: up to 64 rows the
    hand-written weight-streaming kernels (on the packed copy of w when there is one: `packed`),
    up to 128 rows too where w is much longer than it has rows (see long_inner); for more rows the
    hand-written tiled product where it was measured ahead (see tiles_plan); otherwise the
    library product (as the reference uses a library for its prompt products,
    Daisi.Llogos.Cuda/CudaBackend.cs:158-316)."""
    M = a.shape[-2]
    if packed is not None and packed.gate_rows:
        packed = None                                       # its rows are in another order: only the gated product reads it
    if packed is not None and w.dtype == torch.bfloat16 and M <= SKINNY_MAX_ROWS and out_dtype == torch.bfloat16:
        splits, chunk = packed_plan(M, packed.N, packed.K)
        src, fused = a, swiglu_input
        # silu(gate) * up inside the product costs every block of rows of w a second read of the
        # gate/up row: worth it for few rows in bfloat16, not for partial sums or many rows
        if fused and not (M <= 16 and a.dtype == torch.bfloat16 and (a.dim() == 2 or a.shape[0] == 1)):
            src, fused = swiglu(a, out_dtype), False
        if not fused and src.dim() == 3 and src.shape[0] == 1:
            src = src[0]
        out = gemm_packed_bf16(src, packed, None, torch.float32 if f32_ok else out_dtype, splits, chunk, fused)
        if out is not None:
            return out
    if w.dtype == torch.bfloat16 and M <= SKINNY_MAX_ROWS and out_dtype == torch.bfloat16:
        few_dtype = torch.float32 if f32_ok else out_dtype              # what a product in one part is written as
        kernel, splits, row_blocks = skinny_plan(M, w.shape[0], w.shape[1])
        if kernel == "stationary" and not swiglu_input and a.dim() == 2:
            out = gemm_skinny_stationary_bf16(a, w, None, few_dtype, row_blocks)
            if out is not None:
                return out
            kernel, splits, row_blocks = "lds", 1, 1
        elif kernel == "stationary":
            kernel, splits, row_blocks = "lds", 1, 1
        if kernel == "strips":
            if swiglu_input:
                a, swiglu_input = swiglu(a, out_dtype), False
            out = gemm_strips_bf16(a, w, None, few_dtype, splits, row_blocks) if a.dim() == 2 else None
            if out is not None:
                return out
            kernel, splits, row_blocks = "lds", lds_splits(M, w.shape[0], w.shape[1]), 1
        # silu(gate) * up inside the product costs every block of rows of w a second read of the
        # gate/up row: worth it for few rows in bfloat16, not for partial sums or many rows
        if swiglu_input and not (M <= 16 and a.dtype == torch.bfloat16 and (a.dim() == 2 or a.shape[0] == 1)):
            a, swiglu_input = swiglu(a, out_dtype), False
        if swiglu_input or kernel == "lds":
            out = gemm_skinny_lds_bf16(a, w, None, few_dtype, splits if kernel == "lds" else 1, row_blocks,
                                       swiglu_input)
            if out is not None:
                return out
        if not swiglu_input and a.dtype == torch.bfloat16:
            out = gemm_skinny_bf16(a, w, None, few_dtype, splits if kernel == "regs" else 1, row_blocks)
            if out is not None:
                return out
    if swiglu_input:
        a = swiglu(a, out_dtype)
    if SKINNY_MAX_ROWS < M <= LDS_MAX_ROWS and long_inner(w) and a.dtype == torch.bfloat16 and out_dtype == torch.bfloat16:
        out = gemm_skinny_lds_bf16(a, w, None, torch.float32 if f32_ok else out_dtype,
                                   lds_splits(M, w.shape[0], w.shape[1]), 1)
        if out is not None:
            return out
    plan = tiles_plan(M, packed.N, packed.K) if packed is not None else None
    if plan is not None and out_dtype == torch.bfloat16 and a.dtype == torch.bfloat16 and a.dim() == 2:
        out = gemm_tiles_bf16(a, packed, None, torch.float32 if f32_ok else out_dtype, parts=plan[0], token_tiles=plan[1])
        if out is not None:
            return out
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out_dtype == torch.bfloat16 and a.is_contiguous() \
            and M > SKINNY_MAX_ROWS:
        if f32_ok:
            return torch.mm(a, w.t(), out_dtype=torch.float32)
        return torch.matmul(a, w.t())
    return gemm_generic(a, w, None, out_dtype)


def gemm_library_add(x: torch.Tensor, a: torch.Tensor, w: torch.Tensor, packed: Optional[PackedWeight] = None) -> bool:
    """x [M, N] (float32, in place) += a [M, K] . w^T by the library's bfloat16 product with float32
    accumulation and the sum in its epilogue, where the library serves this product anyway (prompts of
    more than 128 rows that the tiled product does not take): the stream is read and written once there
    instead of the product being written, read again and added by the norm's kernel.  False (and x
    untouched) otherwise.  The result is the float32 product added to x, bit for bit."""
    if RESIDUAL_PRODUCT != "on":
        return False
    if not (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dtype == torch.float32 and a.dim() == 2
            and x.dim() == 2 and a.is_contiguous() and x.is_contiguous() and w.is_contiguous()):
        return False
    M, N = a.shape[0], w.shape[0]
    if M <= LDS_MAX_ROWS or x.shape != (M, N) or a.shape[1] != w.shape[1] or a.shape[1] % 8:
        return False
    if packed is not None and tiles_plan(M, packed.N, packed.K) is not None:
        return False
    torch.addmm(x, a, w.t(), out_dtype=torch.float32, out=x)
    return True


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out_dtype: torch.dtype,
         packed: Optional[PackedWeight] = None) -> torch.Tensor:
    """a [M, K] . w [N, K]^T (+ bias [N]) -> one plain [M, N] tensor of `out_dtype`."""
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        M = a.shape[0]
        if packed is not None and not packed.gate_rows and M <= SKINNY_MAX_ROWS:
            out = gemm_packed_bf16(a, packed, bias, out_dtype, 1, packed_plan(M, packed.N, packed.K)[1])
            if out is not None:
                return out[0]
        if M <= SKINNY_MAX_ROWS:
            kernel, _, row_blocks = skinny_plan(M, w.shape[0], w.shape[1])
            if kernel == "stationary":
                out = gemm_skinny_stationary_bf16(a, w, bias, out_dtype, row_blocks)
                kernel, row_blocks = "lds", 1
            elif kernel == "strips":
                out = gemm_strips_bf16(a, w, bias, out_dtype, 1, row_blocks)
                kernel, row_blocks = "lds", 1
            else:
                out = None
            if out is None:
                fn = gemm_skinny_lds_bf16 if kernel == "lds" else gemm_skinny_bf16
                out = fn(a, w, bias, out_dtype, 1, row_blocks)
            if out is not None:
                return out[0]
        elif out_dtype == torch.bfloat16 and a.is_contiguous():
            out = torch.matmul(a, w.t())
            if bias is not None:
                out += bias.to(torch.bfloat16)
            return out
        elif out_dtype == torch.float32 and a.is_contiguous() and a.shape[1] % 8 == 0:
            # float32 results for many rows (the logits of many positions): the library's product
            # with float32 accumulation and output, one pass over w
            out = torch.mm(a, w.t(), out_dtype=torch.float32)
            if bias is not None:
                out += bias
            return out
    return gemm_generic(a, w, bias, out_dtype)


_attn_workspaces = {}
PREFILL_TILE_ROWS = 0        # 0: chosen by the step; 64 or 128 force a prefill attention kernel (tests)
PREFILL_HALVES = 0           # 0: chosen by the step; 1 or 2 sets of waves a block of the 128-row kernel (tests)


def prefill_halves(lens: Sequence[int], starts: Optional[Sequence[int]], n_heads: int, n_cus: Optional[int] = None) -> int:
    """Sets of waves a block of the 128-row prompt attention: 2 (the sets take a tile's pages in
    turn) where the pages of the longest tile, one after the other, take longer than the chip
    needs for all tiles; 1 (two independent blocks a compute unit, 15 % more throughput) where
    the work of all tiles decides.  Measured at the 8B head shape: two sets win up to 2,048
    tokens of one prompt (1,536: 45 us against 57) and lose from 2,560 on and for many short
    prompts."""
    n_cus = n_cus or compute_units()
    longest = total = 0
    for i, n in enumerate(lens):
        start = starts[i] if starts else 0
        for t in range(0, n, 128):
            pages = (start + min(n, t + 128) + PAGE_TOKENS - 1) // PAGE_TOKENS
            longest = max(longest, pages)
            total += pages
    return 2 if longest * 2 * n_cus > 1.7 * total * n_heads else 1


def _attn_workspace(device: torch.device, floats: int) -> torch.Tensor:
    """Scratch memory of the decode attention, at least `floats` long.  A workspace that has
    become too small stays alive beside its successor: captured steps keep its address."""
    key = (device.type, device.index)
    held = _attn_workspaces.setdefault(key, [])
    if not held or held[-1].numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("attention workspace must be made before a step is captured")
        size = max(floats, 1 << 20, 2 * held[-1].numel() if held else 0)
        held.append(torch.empty(size, dtype=torch.float32, device=device))
    return held[-1]


def attention_mfma_bf16(ctx, q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                        table: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                        window: int = 0, sinks: int = 0) -> Optional[torch.Tensor]:
    """bfloat16 attention on the matrix cores; None for shapes it does not take (head sizes
    other than 64 and 128, more than 16 query heads per kv head)."""
    if q.dtype != torch.bfloat16 or head_dim not in (64, 128) or n_heads // n_kv_heads > 16:
        return None
    if q_stride % 8 or q.data_ptr() % 16:
        return None
    _dev(k_pool, v_pool, table)
    _i32(table, "table")
    _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "attention")
    _need(k_pool.dtype == torch.bfloat16, "attention: q and cache types differ")
    T = ctx.n_tokens
    _need(q.numel() >= (T - 1) * q_stride + n_heads * head_dim, "attention: q too small")
    out = torch.empty((T, n_heads * head_dim), dtype=torch.bfloat16, device=q.device)
    lib = _lib()
    if ctx.is_decode:
        width = table.shape[1]
        floats = lib.llogos_attn_decode_workspace(T, n_heads, n_kv_heads, head_dim, width)
        ws = _attn_workspace(q.device, floats)
        code = lib.llogos_attn_decode_bf16(
            _p(out), _p(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0), width, _p(ctx.tok_pos),
            T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks, _p(ws),
            ctypes.c_longlong(ws.numel()), _stream())
    else:
        cu = ctx.cu_dev
        _need(cu is not None and cu.numel() == ctx.batch + 1, "attention: the step's token offsets are missing")
        # long sequences: tiles of 128 tokens whose waves share each page through LDS; short
        # ones: tiles of 64 whose waves read the pages themselves
        lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
        tile_rows = PREFILL_TILE_ROWS or (128 if max(lens) > 64 else 64)
        n_tiles = sum(-(-n // tile_rows) for n in lens)
        halves = PREFILL_HALVES or (prefill_halves(lens, getattr(ctx, "starts", None), n_heads) if tile_rows == 128 else 1)
        code = lib.llogos_attn_prefill_bf16(
            _p(out), _p(q), q_stride, _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(cu), _p(ctx.tok_pos),
            ctx.batch, n_tiles, tile_rows, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks,
            halves, _stream())
    if code == -2:
        return None
    _check(code, "attention_mfma_bf16")
    return out


def attention_decode_fused(ctx, qkv: torch.Tensor, bias: Optional[torch.Tensor], n_heads: int, n_kv_heads: int,
                           head_dim: int, rot: int, pairing: int, q_norm_w: Optional[torch.Tensor],
                           k_norm_w: Optional[torch.Tensor], eps: float, cs: torch.Tensor, k_pool: torch.Tensor,
                           v_pool: torch.Tensor, table: torch.Tensor, scale: float, window: int = 0,
                           sinks: int = 0) -> Optional[torch.Tensor]:
    """A single-token step's attention straight from the fused projection rows [q | k | v]
    (float32 [T, W] or partial sums [parts, T, W]): bias, per-head norm, rotation and the cache
    write happen inside the attention kernel.  For bfloat16 caches, head sizes 64 and 128 rotated
    whole with split-half pairing; None for anything else (the caller then runs the steps apart)."""
    if not (ctx.is_decode and qkv.dtype == torch.float32 and k_pool.dtype == torch.bfloat16 and head_dim in (64, 128)
            and rot == head_dim and pairing == 0 and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16):
        return None
    parts, part_stride = _parts(qkv)
    T = qkv.shape[-2]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    if qkv.stride(-1) != 1 or qkv.stride(-2) % 2 or part_stride % 2 or qkv.data_ptr() % 8:
        return None
    _dev(qkv, bias, q_norm_w, k_norm_w, cs, k_pool, v_pool, table, ctx.tok_pos)
    _i32(table, "table"); _i32(ctx.tok_pos, "tok_pos")
    _need(T == ctx.n_tokens == ctx.batch and qkv.shape[-1] == width, f"attention: qkv must be [{ctx.batch}, {width}]")
    _need(cs.dtype == torch.float32 and cs.shape == (T, rot // 2, 2) and cs.is_contiguous(), "attention: rotary table shape")
    _need(table.dim() == 2 and table.shape[0] == T and ctx.tok_pos.numel() == T, "attention: one table row and position a sequence")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (width,), f"attention: bias must be float32 [{width}]")
    for wgt in (q_norm_w, k_norm_w):
        if wgt is not None:
            _need(wgt.dtype == torch.float32 and wgt.shape == (head_dim,), "attention: norm weight float32 [head_dim]")
    _check_pools(k_pool, v_pool, n_kv_heads, head_dim, "attention")
    _need(v_pool.dtype == torch.bfloat16, "attention: cache types differ")
    out = torch.empty((T, n_heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    lib = _lib()
    width_pages = table.shape[1]
    ws = _attn_workspace(qkv.device, lib.llogos_attn_decode_workspace(T, n_heads, n_kv_heads, head_dim, width_pages))
    code = lib.llogos_attn_decode_fused_bf16(
        _p(out), _p(qkv), parts, ctypes.c_longlong(part_stride), qkv.stride(-2), _p(bias), _p(q_norm_w), _p(k_norm_w),
        ctypes.c_float(eps), _p(cs), _p(k_pool), _p(v_pool), _p(table), table.stride(0), width_pages, _p(ctx.tok_pos),
        T, n_heads, n_kv_heads, head_dim, ctypes.c_float(scale), window, sinks, _p(ws),
        ctypes.c_longlong(ws.numel()), _stream())
    if code == -2:
        return None
    _check(code, "attention_decode_fused")
    return out


def attention(ctx, q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
              table: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
              window: int = 0, sinks: int = 0) -> torch.Tensor:
    """Attention of the step's query rows over the cache pages of their sequences."""
    if q.dtype == torch.bfloat16:
        out = attention_mfma_bf16(ctx, q, q_stride, k_pool, v_pool, table, n_heads, n_kv_heads, head_dim, scale,
                                  window, sinks)
        if out is not None:
            return out
    return attention_generic(q, q_stride, k_pool, v_pool, table, ctx.tok_seq, ctx.tok_pos,
                             n_heads, n_kv_heads, head_dim, scale, window, sinks)


CAPPED_PREFILL_TILE_ROWS = 0      # 0: chosen by the step; 64 or 128 force a prompt kernel of the attention with bent scores (tests)
CAPPED_PREFILL_HALVES = 0         # 0: chosen by the step; 1 or 2 sets of waves a block of the 128-row kernel (tests)


def capped_attention(ctx, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, table: torch.Tensor, n_heads: int,
                     n_kv_heads: int, head_dim: int, v_dim: int, scale: float, softcap: float = 0.0,
                     head_sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of the step's query rows q [T, n_heads * head_dim] over their sequences' pages, for keys of
    head_dim and values of v_dim dimensions: scores bent to softcap * tanh(score / softcap) (softcap > 0), a sink in
    the softmax's denominator (head_sink float32 [n_heads]: exp(head_sink[h]) is added to head h's sums; zeros for a
    sink of score 0), head h's output times
    sigmoid(gate[t, h]) (gate float32 [T, >= n_heads], maybe a view of wider rows).  Returns [T, n_heads * v_dim].
    bfloat16 with head sizes the matrix-core kernels take runs there; everything else in the kernel for any shape."""
    T = ctx.n_tokens
    if q.dtype == torch.bfloat16 and q.dim() == 2 and q.is_contiguous():
        kd, vd = _page_dims(k_pool, v_pool, n_kv_heads, "attention")
        if kd == head_dim and vd == v_dim and v_pool is not None:
            _dev(table, ctx.tok_pos)
            _i32(table, "table")
            _need(tuple(q.shape) == (T, n_heads * head_dim), "attention: q must be [T, heads * head_dim]")
            gate_stride = 0
            if gate is not None:
                _need(gate.is_cuda and gate.dtype == torch.float32 and gate.dim() == 2 and gate.shape[0] == T
                      and gate.shape[1] >= n_heads and gate.stride(1) == 1, "attention: gate must be float32 [T, n_heads]")
                gate_stride = gate.stride(0) if T > 1 else max(n_heads, gate.stride(0))
            out = torch.empty((T, n_heads * v_dim), dtype=torch.bfloat16, device=q.device)
            lib = _lib()
            if head_sink is not None:
                _dev(head_sink)
                _need(head_sink.dtype == torch.float32 and head_sink.shape == (n_heads,), "attention: head_sink must be float32 [n_heads]")
            if ctx.is_decode:
                width = table.shape[1]
                _need(table.shape[0] == T and ctx.tok_pos.numel() == T, "attention: one table row and position a sequence")
                ws = _attn_workspace(q.device, lib.llogos_capped_attn_decode_workspace(T, n_heads, n_kv_heads, v_dim, width))
                code = lib.llogos_capped_attn_decode_bf16(
                    _p(out), _p(q), q.stride(0), _p(k_pool), _p(v_pool), _p(table), table.stride(0), width, _p(ctx.tok_pos), T,
                    n_heads, n_kv_heads, head_dim, v_dim, ctypes.c_float(scale), ctypes.c_float(softcap), _p(head_sink), _p(gate),
                    gate_stride, _p(ws), ctypes.c_longlong(ws.numel()), _stream())
            else:
                cu = ctx.cu_dev
                _need(cu is not None and cu.numel() == ctx.batch + 1, "attention: the step's token offsets are missing")
                # long sequences: tiles of 128 tokens whose pages go straight into LDS once for a block's waves (the
                # dense decoder's prompt kernel with the bent softmax); short ones: tiles of 64 whose waves read the pages
                lens = [ctx.cu_seqlens[i + 1] - ctx.cu_seqlens[i] for i in range(ctx.batch)]
                tile_rows = CAPPED_PREFILL_TILE_ROWS or (128 if max(lens) > 64 else 64)
                n_tiles = sum(-(-n // tile_rows) for n in lens)
                halves = CAPPED_PREFILL_HALVES or (prefill_halves(lens, getattr(ctx, "starts", None), n_heads) if tile_rows == 128 else 1)
                code = lib.llogos_capped_attn_prefill_bf16(
                    _p(out), _p(q), q.stride(0), _p(k_pool), _p(v_pool), _p(table), table.stride(0), _p(cu), _p(ctx.tok_pos),
                    ctx.batch, n_tiles, n_heads, n_kv_heads, head_dim, v_dim, ctypes.c_float(scale), ctypes.c_float(softcap),
                    _p(head_sink), _p(gate), gate_stride, int(tile_rows), int(halves), _stream())
            if code != -2:
                _check(code, "capped_attention")
                return out
    return attention_generic(q, n_heads * head_dim, k_pool, v_pool, table, ctx.tok_seq, ctx.tok_pos, n_heads, n_kv_heads,
                             head_dim, scale, v_dim=v_dim, head_sink=head_sink, softcap=softcap, gate=gate)


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------
def sample_prepare(logits: torch.Tensor, history: Optional[torch.Tensor], history_len: Optional[torch.Tensor],
                   repetition: float, frequency: float, presence: float, temperature: float,
                   penalize_newline: bool, banned: Sequence[int] = ()) -> torch.Tensor:
    """A copy of float32 logits [R, V] with penalties over each row's recent tokens
    (`history` int32 [R, W], `history_len` int32 [R]), banned ids at -inf, times 1/temperature."""
    _dev(logits, history, history_len)
    _i32(history, "history"); _i32(history_len, "history_len")
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "sample_prepare: logits must be float32 [R, V]")
    _need(len(banned) <= MAX_BANNED, f"sample_prepare: at most {MAX_BANNED} banned ids, got {len(banned)}")
    R, V = logits.shape
    if history is not None:
        _need(history.dim() == 2 and history.shape[0] == R and history_len is not None
              and history_len.numel() == R, "sample_prepare: history [R, W] with lengths [R]")
    work = torch.empty_like(logits)
    ban = (ctypes.c_int * MAX_BANNED)(*list(banned))
    inv_t = 1.0 / temperature if temperature > 0 else 1.0
    _check(_lib().llogos_sample_prepare(
        _p(work), _p(logits), R, V, _p(history), _p(history_len), history.stride(0) if history is not None else 0,
        ctypes.c_float(repetition), ctypes.c_float(frequency), ctypes.c_float(presence), ctypes.c_float(inv_t),
        int(penalize_newline), ban, len(banned), _stream()), "sample_prepare")
    return work


SAMPLE_ORDERS = {"single": 0, "head": 1, "whole": 2}


def sample_pipeline(work: torch.Tensor, uniforms: torch.Tensor, top_k: int, top_p: float, min_p: float,
                    typical_p: float, min_keep: int, order: str = "head") -> torch.Tensor:
    """Token ids int32 [R] drawn from prepared rows `work` with one uniform number per row:
    top-k, min-p, softmax, typical-p, top-p, draw.  order "head": a row is first tried with
    the head of its descending order alone (a histogram finds it; no sort of the vocabulary),
    and rows that this cannot decide are sorted whole by many blocks; "whole": every row is
    sorted so; "single": every row is sorted by its own block (slow, the plain form).  Rows
    sorted whole are overwritten with probabilities."""
    _dev(work, uniforms)
    _need(work.dtype == torch.float32 and work.dim() == 2, "sample_pipeline: work must be float32 [R, V]")
    _need(order in SAMPLE_ORDERS, f"sample_pipeline: order must be one of {sorted(SAMPLE_ORDERS)}")
    R, V = work.shape
    _need(uniforms.dtype == torch.float32 and uniforms.numel() == R, "sample_pipeline: one float32 uniform per row")
    n_pad = 1
    while n_pad < V:
        n_pad <<= 1
    scratch = torch.empty((R, n_pad), dtype=torch.int64, device=work.device)
    prob = torch.empty_like(work) if order == "head" else None
    out = torch.empty((R,), dtype=torch.int32, device=work.device)
    _check(_lib().llogos_sample_pipeline(
        _p(out), _p(work), _p(prob), R, V, _p(scratch), n_pad, _p(uniforms), int(top_k), ctypes.c_float(top_p),
        ctypes.c_float(min_p), ctypes.c_float(typical_p), int(min_keep), SAMPLE_ORDERS[order], _stream()),
        "sample_pipeline")
    return out


# ----------------------------------------------------------------------------
# what the GPU does at best, measured
# ----------------------------------------------------------------------------
def measure_read_bandwidth(n_bytes: int, repeats: int = 20, blocks_per_unit: int = 8, device="cuda:0") -> float:
    """Bytes a second at which a kernel that only reads streams `n_bytes` of device memory
    (16-byte loads that do not stay in the caches, 32 KB of consecutive memory a block and round),
    best of `repeats` runs over a buffer that was not the last thing read."""
    dev = torch.device(device)
    n_bytes = max(1 << 20, n_bytes // 16 * 16)
    with torch.cuda.device(dev):
        buf = torch.empty(n_bytes // 4, dtype=torch.int32, device=dev).fill_(1)
        other = torch.empty(max(n_bytes // 4, 1 << 27), dtype=torch.int32, device=dev).fill_(2)   # evicts the caches
        sink = torch.zeros(4, dtype=torch.int32, device=dev)
        blocks = compute_units(dev) * blocks_per_unit
        lib, best = _lib(), 0.0
        for _ in range(repeats):
            _check(lib.llogos_measure_read(_p(other), ctypes.c_longlong(other.numel() * 4), blocks, _p(sink), _stream()), "measure_read")
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            _check(lib.llogos_measure_read(_p(buf), ctypes.c_longlong(n_bytes), blocks, _p(sink), _stream()), "measure_read")
            end.record()
            end.synchronize()
            best = max(best, n_bytes / (start.elapsed_time(end) * 1e-3))
    return best


def measure_mfma_rate(iters: int = 20000, blocks_per_unit: int = 2, device="cuda:0", noisy: bool = True,
                      shapes=(16, 32)) -> float:
    """bfloat16 flops a second of MFMAs issued back to back by eight waves on every compute unit
    (independent accumulators): the better of v_mfma_f32_16x16x32_bf16 and v_mfma_f32_32x32x16_bf16.
    noisy: operands of random values, as real data is (the chip clocks lower under their power than
    with the few small constants of noisy=False)."""
    dev = torch.device(device)
    with torch.cuda.device(dev):
        blocks = compute_units(dev) * blocks_per_unit
        out = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
        lib, best = _lib(), 0.0
        for shape in tuple(shapes) * 2:
            per_iter = 8 * 16384.0 if shape == 16 else 4 * 32768.0
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            _check(lib.llogos_measure_mfma(_p(out), blocks, iters, shape, int(noisy), _stream()), "measure_mfma")
            end.record()
            end.synchronize()
            best = max(best, blocks * 4 * iters * per_iter / (start.elapsed_time(end) * 1e-3))
    return best
