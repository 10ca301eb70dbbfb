"""The Zasidra design on the GPU against the plain implementation: every mechanism alone, whole
prompts, prompts cut into portions, token-by-token decoding, unequal batches with slots and pages
used again, long decoding over page borders, sensitivity to a far key, to the sink, to the rotation's
stretch and to another layer's keys, greedy generation through the library's entry point, and the
trace runner and the command line as programs."""
import importlib
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_zasidra as pz
import zasidra_configs as zc
import zasidra_helpers as H

pytestmark = pytest.mark.gpu
L = H.llogos
P = importlib.import_module("daisi-llogos_amd.parts")
K = importlib.import_module("daisi-llogos_amd.ops.kernels")
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
PART_TOL = {"float32": 3e-5, "bfloat16": 3e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _np(t):
    return t.detach().cpu().double().numpy()


def _i32(a):
    return torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)


def _rounded(a, dtype):
    """Random inputs as the engine's type holds them, as float64."""
    return np.asarray(torch.tensor(a).to(DT[dtype]).double())


def _ctx(rt, lens, new, slots):
    """A step that brings new[i] tokens to sequence i, which is lens[i] long afterwards."""
    B, T = len(lens), sum(new)
    tok_seq = np.repeat(np.arange(B), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    cu = np.concatenate([[0], np.cumsum(new)])
    return P.StepContext(runtime=rt, n_tokens=T, batch=B, ids=_i32(np.zeros(T)), tok_seq=_i32(tok_seq),
                         tok_pos=_i32(tok_pos), slots=_i32(slots), cu_seqlens=cu.tolist(), starts=[l - n for l, n in zip(lens, new)],
                         slot_ids=list(slots), is_decode=max(new) == 1, max_context=max(lens),
                         cu_dev=None if max(new) == 1 else _i32(cu))


def _steps(lengths, cuts):
    """Cut sequences of `lengths` into steps: cuts[s][i] tokens of sequence i in step s (0: not in the step)."""
    done = [0] * len(lengths)
    for cut in cuts:
        seqs = [i for i, c in enumerate(cut) if c]
        lo = [done[i] for i in seqs]
        for i in seqs:
            done[i] += cut[i]
        yield seqs, lo, [done[i] for i in seqs]
    assert done == list(lengths), "the cuts do not cover the sequences"


def _bind(part, rng, dtype, scale=0.3, scaled=None):
    """Random tensors for a part (stored in bfloat16, as a model folder holds them); returns them as float64."""
    tensors, plain = {}, {}
    lim = {"norm": (0.7, 1.3), "offset": (-0.3, 0.3), "sink": (0.0, 3.0), "router": (-0.4, 0.4), "correction": (-0.15, 0.15)}
    for spec in part.tensor_specs():
        if spec.kind in lim:
            t = torch.tensor(rng.uniform(*lim[spec.kind], size=spec.shape), dtype=torch.bfloat16)
        else:
            t = torch.tensor(rng.standard_normal(spec.shape) * scale * (scaled or {}).get(spec.name, 1.0), dtype=torch.bfloat16)
        tensors[spec.name], plain[spec.name] = t, t.double().numpy()
    part.bind(tensors.get, P.Runtime(DEV, DT[dtype]))
    return plain


def _rebind(part, plain, dtype):
    part.bind({k: torch.tensor(v, dtype=torch.bfloat16) for k, v in plain.items()}.get, P.Runtime(DEV, DT[dtype]))


def _run(eng, slot, toks, lo, hi):
    return eng.step([(slot, list(toks[lo:hi]))], want="all")


# ---------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("width", [6, 70, 256, 1000, 5000])
@pytest.mark.parametrize("rows", ["float32", "bfloat16"])
def test_the_closing_kernel_norms_the_output_adds_it_and_leaves_the_rows(width, rows):
    rng = np.random.default_rng(width)
    T = 5
    x = rng.standard_normal((T, width)) * 3 + 1.5
    parts = rng.standard_normal((3, T, width))
    w = rng.uniform(0.5, 1.5, size=width)
    f = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    want = x + pz.plain_norm(parts.sum(0), w, 1e-5)
    xt = f(x)
    got = K.sandwich_norm(xt, f(parts), f(w), None, 1e-5, DT[rows], plain_rows=True)
    assert np.abs(_np(xt) - want).max() <= 2e-5 * np.abs(want).max()
    assert got.dtype == DT[rows] and np.abs(_np(got) - want).max() <= (2e-5 if rows == "float32" else 1e-2) * np.abs(want).max()
    xt = f(x)
    assert K.sandwich_norm(xt, f(parts[0]).to(DT[rows]), f(w), None, 1e-5, DT[rows]) is None        # the stream alone
    want = x + pz.plain_norm(_np(f(parts[0]).to(DT[rows])), w, 1e-5)
    assert np.abs(_np(xt) - want).max() <= 2e-5 * np.abs(want).max()


def _closing(kind, y, w, eps):
    if kind == "rms":
        return pz.offset_norm(y, w, eps)
    y = np.asarray(y, dtype=np.float64)                        # a layer norm with a weight and no bias
    d = y - y.mean(axis=-1, keepdims=True)
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + eps) * w


@pytest.mark.parametrize("kind", ["rms", "layer"])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_a_block_of_the_design_with_toy_parts(dtype, kind):
    """x + N1(mixer(x)), then + N2(ff(x)), with a dense feed-forward; the closing norms are the design's own (one kernel
    closes a sublayer) or norms of another kind (their own kernel, then a sum)."""
    rng = np.random.default_rng(3)
    W, T = 40, 7
    if kind == "rms":
        norm = lambda n: P.RMSNorm(name=n, width=W, eps=1e-5, offset=1.0, suffix="")
    else:
        norm = lambda n: P.LayerNorm(name=n, width=W, eps=1e-5, suffix="")
    ff = P.SwiGLU(prefix="f.", hidden=W, intermediate=24, names=("gate", "up", "down"), suffix="")

    class Doubler(P.Mixer):                                    # a mixer without tensors: twice its input
        def forward(self, ctx, h, cache):
            return (h.float() * 2.0).to(h.dtype)
    blk = P.OutputNormBlock(mixer_norm=norm("n1"), mixer=Doubler(), ffn_norm=norm("n2"), ffn=ff)
    plain = _bind(blk, rng, dtype)
    x = _rounded(rng.standard_normal((T, W)), "float32")
    xt = torch.tensor(x, dtype=torch.float32, device=DEV)
    out, pending = blk.forward(None, xt, None, [P.LayerCache()])
    h = _rounded(x, dtype)
    want = x + _closing(kind, 2.0 * h, plain["n1"], 1e-5)
    want = want + _closing(kind, pz.gated_ff(_rounded(want, dtype), plain["f.gate"], plain["f.up"], plain["f.down"]), plain["n2"], 1e-5)
    assert np.abs(_np(out) - want).max() <= PART_TOL[dtype] * np.abs(want).max()
    if dtype == "float32":
        assert pending is None
    else:
        assert pending.norm is None and np.abs(_np(pending.rows) - want).max() <= 1e-2 * np.abs(want).max()


# (heads, kv heads, key width, value width, hidden, rotated width, stretched)
ATTENTIONS = [(4, 2, 32, 48, 56, 16, True), (3, 3, 24, 40, 64, 24, False), (5, 1, 8, 16, 40, 0, False), (2, 1, 64, 80, 64, 32, True),
              (4, 2, 96, 64, 96, 64, False), (2, 2, 128, 128, 64, 128, True), (16, 1, 64, 64, 32, 2, True), (4, 2, 64, 128, 48, 32, False)]


def _rotary(dim, rot_dims, stretched):
    if not rot_dims:
        return None, None
    scaling = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0} if stretched else None
    lib = dict(scaling, type="yarn") if scaling else None
    return P.Rotary(dim, rot_dims, 3000.0, pairing="split_half", scaling=lib), {"dims": rot_dims, "base": 3000.0, "scaling": scaling}


def _attention(shape, own_kv=True, scale=0.2):
    heads, kv, dk, dv, hidden, rot_dims, stretched = shape
    position, rot = _rotary(dk, rot_dims, stretched)
    mix = P.CappedAttention(prefix="m.", hidden=hidden, n_heads=heads, n_kv_heads=kv, head_dim=dk, v_dim=dv, scale=scale, eps=1e-5,
                            whole_norm=True, learned_sink=True, position=position, own_kv=own_kv)
    m = {"heads": heads, "kv_heads": kv, "dim": dk, "vdim": dv, "scale": scale, "rot": rot}
    return mix, m


@pytest.mark.parametrize("dtype,tile_rows,halves", [("float32", 0, 0), ("bfloat16", 0, 0), ("bfloat16", 64, 1), ("bfloat16", 128, 1),
                                                    ("bfloat16", 128, 2)])
@pytest.mark.parametrize("shape", ATTENTIONS)
def test_the_attention_and_a_reader_of_its_keys_alone_in_pieces(dtype, tile_rows, halves, shape, monkeypatch):
    """Three sequences cut into steps of several sizes, their pages in any order, a page of NaN that nobody may
    read; an owner of keys and values, and behind it a second mixer that reads the owner's pages with queries,
    sink and output matrix of its own.  Shapes that the matrix-core kernels take must run there in bfloat16."""
    heads, kv, dk, dv, hidden, rot_dims, stretched = shape
    monkeypatch.setattr(K, "CAPPED_PREFILL_TILE_ROWS", tile_rows)        # every prompt kernel of the matrix cores in turn
    monkeypatch.setattr(K, "CAPPED_PREFILL_HALVES", halves)
    rng = np.random.default_rng(heads * 100 + dk)
    own, m = _attention(shape)
    reader, _ = _attention(shape, own_kv=False)
    assert not any(s.name in ("m.k", "m.v", "m.k.norm") for s in reader.tensor_specs())
    plain = _bind(own, rng, dtype, scaled={"m.q": 2.0, "m.k": 2.0})
    plain_r = _bind(reader, rng, dtype, scaled={"m.q": 2.0})
    lengths = (150, 70, 3)
    h = [_rounded(rng.standard_normal((n, hidden)), dtype) for n in lengths]
    h2 = [_rounded(rng.standard_normal((n, hidden)), dtype) for n in lengths]
    want, want_r = [], []
    for x, x2 in zip(h, h2):
        o, kvs = pz.attention(x, pz.part(plain, "m."), m, 1e-5, np.arange(len(x)))
        want.append(o)
        want_r.append(pz.attention(x2, pz.part(plain_r, "m."), m, 1e-5, np.arange(len(x)), kvs)[0])
    spec = own.kv_spec()
    assert reader.kv_spec() == spec
    k_pool = torch.zeros((9, kv, 64 * spec.head_dim), dtype=DT[dtype], device=DEV)
    v_pool = torch.zeros((9, kv, 64 * spec.value_dim), dtype=DT[dtype], device=DEV)
    k_pool[4] = float("nan"); v_pool[4] = float("nan")
    pages = {0: [7, 2, 5], 1: [0, 8], 2: [3]}
    slots = [1, 3, 0]
    fast = dtype == "bfloat16" and dk in (64, 96, 128) and dv in (64, 80, 96, 128)
    if fast:
        monkeypatch.setattr(K, "attention_generic", lambda *a, **k: pytest.fail("the kernel for any shape ran"))
    got, got_r = [np.zeros((n, hidden)) for n in lengths], [np.zeros((n, hidden)) for n in lengths]
    cuts = [(60, 9, 1), (1, 1, 1), (1, 1, 1), (3, 58, 0), (1, 1, 0), (2, 0, 0), (64, 0, 0), (1, 0, 0), (17, 0, 0)]
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(own.rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        table = np.full((len(seqs), 3), -1, dtype=np.int32)
        for r, i in enumerate(seqs):
            table[r, :len(pages[i])] = pages[i]
        rows = lambda src: torch.tensor(np.concatenate([src[i][a:b] for i, a, b in zip(seqs, lo, hi)]), dtype=DT[dtype], device=DEV)
        cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=_i32(table))
        o = _np(K.sum_parts(own.forward(ctx, rows(h), cache), None, torch.float32))
        cache_r = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=_i32(table), writes=False)
        o_r = _np(K.sum_parts(reader.forward(ctx, rows(h2), cache_r), None, torch.float32))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b], got_r[i][a:b] = o[at:at + b - a], o_r[at:at + b - a]
            at += b - a
    tol = (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype]
    for i in range(3):
        assert np.isfinite(got[i]).all() and np.isfinite(got_r[i]).all()
        assert np.abs(got[i] - want[i]).max() <= tol * max(1.0, np.abs(want[i]).max()), f"owner, sequence {i}"
        assert np.abs(got_r[i] - want_r[i]).max() <= tol * max(1.0, np.abs(want_r[i]).max()), f"reader, sequence {i}"
    with pytest.raises(RuntimeError):                          # a reader that is given pages to write
        reader.forward(ctx, rows(h2), cache)


def test_a_far_key_the_sink_and_the_stretch_decide_in_the_attention_alone():
    """One key far back is made to stand out; without it, without the sink, with a sink of score 0, or with plain
    frequencies the plain result moves by many times the bound, and the kernels agree with the full one."""
    rng = np.random.default_rng(5)
    shape = (2, 1, 64, 80, 64, 32, True)
    mix, m = _attention(shape)
    plain = _bind(mix, rng, "float32", scaled={"m.q": 3.0, "m.k": 3.0})
    t = pz.part(plain, "m.")
    n = 330
    h = rng.standard_normal((n, 64))
    h[3] *= 4.0                                                               # a loud early token: its key stands out for many queries
    pos = np.arange(n)
    want, (k, v) = pz.attention(h, t, m, 1e-5, pos)
    k2 = k.copy(); k2[3] = 0.0
    no_key = pz.attention(h, t, m, 1e-5, pos, (k2, v))[0]
    no_sink = pz.attention(h, dict(t, sink=np.full(2, -1e9)), m, 1e-5, pos)[0]
    unit_sink = pz.attention(h, dict(t, sink=np.zeros(2)), m, 1e-5, pos)[0]
    plain_rot = pz.attention(h, t, dict(m, rot=dict(m["rot"], scaling=None)), 1e-5, pos)[0]
    whole_rot = pz.attention(h, t, dict(m, rot=dict(m["rot"], dims=64)), 1e-5, pos)[0]
    size = np.abs(want).max()
    for other in (no_key[300:], plain_rot[300:], whole_rot[300:]):
        assert np.abs(other - want[300:]).max() > 100 * PART_TOL["float32"] * size
    for other in (no_sink, unit_sink):
        assert np.abs(other - want).max() > 100 * PART_TOL["float32"] * size
    for dtype in H.DTYPES:
        mix, _ = _attention(shape)
        _rebind(mix, plain, dtype)
        k_pool = torch.zeros((6, 1, 64 * 64), dtype=DT[dtype], device=DEV)
        v_pool = torch.zeros((6, 1, 64 * 80), dtype=DT[dtype], device=DEV)
        table = _i32([[4, 1, 0, 5, 2, 3]])
        got = []
        for lo, hi in [(0, 257)] + [(t_, t_ + 1) for t_ in range(257, n)]:
            ctx = _ctx(mix.rt, [hi], [hi - lo], [0])
            cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=table)
            got.append(_np(K.sum_parts(mix.forward(ctx, torch.tensor(h[lo:hi], dtype=DT[dtype], device=DEV), cache), None, torch.float32)))
        assert np.abs(np.concatenate(got) - want).max() <= PART_TOL[dtype] * size * (1 if dtype == "float32" else 3)


# (heads, key width, value width, rank, hidden)
LATENTS = [(3, 24, 40, 48, 56), (5, 16, 8, 20, 40), (2, 40, 24, 24, 72), (4, 64, 64, 64, 64), (2, 128, 96, 128, 96), (20, 32, 32, 256, 64),
           (1, 8, 8, 8, 16)]


PIECES = [(60, 9, 1), (1, 1, 1), (1, 1, 1), (3, 58, 0), (1, 1, 0), (2, 0, 0), (64, 0, 0), (1, 0, 0), (17, 0, 0)]
WHOLE = [(148, 68, 3), (1, 1, 0), (1, 1, 0)]          # prompts whole in one step (keys and values a head where the shapes allow), then single tokens


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("cuts", [PIECES, WHOLE])
@pytest.mark.parametrize("shape", LATENTS)
def test_the_gated_latent_attention_alone_in_pieces(dtype, shape, cuts, monkeypatch):
    heads, dk, dv, rank, hidden = shape
    rng = np.random.default_rng(heads * 10 + rank)
    # scores that spread over some units whatever the sizes: sharp, and still within what bfloat16 queries resolve
    scale = 6.0 / (0.36 * np.sqrt(float(dk) * hidden * rank))
    mix = P.LatentAttention(prefix="m.", hidden=hidden, n_heads=heads, dim=dk, rot_dim=0, v_dim=dv, q_rank=0, kv_rank=rank, scale=scale,
                            eps=1e-5, sink=False, head_gate=True)
    mix.rt = P.Runtime(DEV, DT[dtype])                         # (the cache's shape depends on the type)
    plain = _bind(mix, rng, dtype, scaled={"m.q": 2.0, "m.uk": 2.0, "m.g": 3.0})
    assert set(plain) == {"m.q", "m.dkv", "m.g", "m.o", "m.dkv.norm", "m.uk", "m.uv"}
    m = {"heads": heads, "dim": dk, "vdim": dv, "kv_rank": rank, "scale": scale}
    lengths = (150, 70, 3)
    h = [_rounded(rng.standard_normal((n, hidden)), dtype) for n in lengths]
    want = [pz.latent_attention(x, pz.part(plain, "m."), m, 1e-5) for x in h]
    spec = mix.kv_spec()
    assert spec.n_kv_heads == 1 and spec.head_dim == -(-rank // 16) * 16
    k_pool = torch.zeros((9, 1, 64 * spec.head_dim), dtype=DT[dtype], device=DEV)
    v_pool = torch.zeros((9, 1, 64 * spec.head_dim), dtype=DT[dtype], device=DEV) if spec.values else None
    k_pool[4] = float("nan")
    if v_pool is not None:
        v_pool[4] = float("nan")
    pages = {0: [7, 2, 5], 1: [0, 8], 2: [3]}
    got = [np.zeros((n, hidden)) for n in lengths]
    by_head = cuts is WHOLE and dtype == "bfloat16" and dk in (64, 96, 128) and dv in (64, 80, 96, 128)
    ran = []
    if by_head:                                                # the whole prompts must take the way over keys and values a head
        keep = mix._forward_prompt
        monkeypatch.setattr(mix, "_forward_prompt", lambda *a, **k: (ran.append(1), keep(*a, **k))[1])
        fresh = torch.empty

        def poisoned(*a, **k):                                 # the step's own pages start as NaN: what is not written is not read
            t = fresh(*a, **k)
            if t.dtype == torch.bfloat16 and t.dim() == 3:
                t.fill_(float("nan"))
            return t
        monkeypatch.setattr(torch, "empty", poisoned)
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(mix.rt, hi, [b - a for a, b in zip(lo, hi)], [0, 1, 2][:len(seqs)])
        table = np.full((len(seqs), 3), -1, dtype=np.int32)
        for r, i in enumerate(seqs):
            table[r, :len(pages[i])] = pages[i]
        cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=_i32(table))
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), dtype=DT[dtype], device=DEV)
        o = _np(K.sum_parts(mix.forward(ctx, rows, cache), None, torch.float32))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.isfinite(g).all()
        assert np.abs(g - w_).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"
    assert len(ran) == (1 if by_head else 0)
    no_gate = pz.latent_attention(h[0], dict(pz.part(plain, "m."), g=np.zeros((heads, hidden))), m, 1e-5)
    assert np.abs(no_gate - want[0]).max() > 100 * PART_TOL["float32"] * np.abs(want[0]).max()      # the gate is no trifle here


@pytest.mark.parametrize("outputs,groups,keep,top,K_,T", [(8, 4, 2, 3, 96, 9), (16, 4, 3, 4, 72, 70), (6, 1, 1, 6, 40, 5), (12, 3, 2, 3, 128, 300),
                                                          (5, 5, 2, 2, 33, 64), (64, 8, 4, 8, 256, 65), (2, 2, 1, 1, 16, 1), (300, 1, 1, 70, 64, 3)])
@pytest.mark.parametrize("rows", H.DTYPES)
def test_the_routers_choice_and_weights(outputs, groups, keep, top, K_, T, rows):
    """Few rows and many (the logits' two kernels), corrections that change the choice, groups of one, all
    groups kept, more choices than a wave has lanes."""
    rng = np.random.default_rng(outputs + top)
    h = _rounded(rng.standard_normal((T, K_)), rows)
    w = _rounded(rng.uniform(-0.4, 0.4, size=(outputs, K_)), "float32")
    c = _rounded(rng.uniform(-0.1, 0.1, size=outputs), "float32")
    r = {"experts": outputs, "top": top, "scale": 1.5, "groups": {"count": groups, "keep": keep} if groups > 1 else None}
    want_c, want_w = pz.route(h, w, c, r)
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    got_c, got_w = K.moe_router(torch.tensor(h, dtype=DT[rows], device=DEV), f32(w), f32(c), groups, keep, top, 1.5)
    got_c, got_w = got_c.cpu().numpy(), _np(got_w)
    close_calls = 0
    for t in range(T):
        if got_c[t].tolist() != want_c[t].tolist():             # equal up to 32-bit rounding of two scores?
            close_calls += 1
            continue
        assert np.abs(got_w[t] - want_w[t]).max() <= 1e-5
    assert close_calls <= max(1, T // 50)
    assert np.abs(got_w.sum(1) - 1.5).max() <= 1e-5
    none_c, _ = K.moe_router(torch.tensor(h, dtype=DT[rows], device=DEV), f32(w), None, groups, keep, top, 1.5)
    assert (none_c.cpu().numpy() != got_c).any() or T * top < 8          # the correction decides somewhere


def test_the_router_refuses_what_it_cannot_choose_from():
    h = torch.zeros((2, 16), dtype=torch.float32, device=DEV)
    w = torch.zeros((6, 16), dtype=torch.float32, device=DEV)
    with pytest.raises(K.KernelError):
        K.moe_router(h, w, None, 3, 1, 3, 1.0)                 # a kept group of two for three choices
    with pytest.raises(K.KernelError):
        K.moe_router(h, w, None, 4, 2, 2, 1.0)                 # groups that do not divide the outputs
    with pytest.raises(K.KernelError):
        K.moe_router(h, w.bfloat16(), None, 1, 1, 2, 1.0)      # a router stored in 16 bits


@pytest.mark.parametrize("dtype,form", [("float32", "auto"), ("bfloat16", "auto"), ("bfloat16", "plain"), ("bfloat16", "few"),
                                        ("bfloat16", "tiles64"), ("bfloat16", "tiles128")])
@pytest.mark.parametrize("experts,identity,groups,keep,top,ff,shared,hidden,T", [
    (6, 2, 4, 2, 3, 40, 24, 96, 9), (1, 1, 1, 1, 1, 16, 8, 32, 3), (4, 0, 1, 1, 4, 24, 0, 48, 70), (8, 4, 3, 2, 3, 72, 136, 64, 300),
    (16, 0, 4, 1, 1, 96, 96, 128, 1), (3, 1, 2, 1, 2, 132, 20, 200, 150), (2, 0, 2, 2, 1, 30, 6, 36, 40), (0, 2, 1, 1, 2, 8, 16, 32, 5)])
def test_the_routed_experts(dtype, form, experts, identity, groups, keep, top, ff, shared, hidden, T, monkeypatch):
    """Every form of the experts' product with its gated epilogue (chosen by the step, or forced: plain multiply-adds, and
    on the matrix cores tiles of 16, 64 and 128 sorted rows); outputs without matrices; no shared expert; no expert
    with matrices at all; the last but one shape has a width that only the plain form takes."""
    monkeypatch.setattr(K, "MOE_PRODUCT", form)
    rng = np.random.default_rng(experts * 10 + top)
    moe = P.RoutedMoE(prefix="f.", hidden=hidden, n_experts=experts, identity=identity, top=top, intermediate=ff, groups=groups, keep=keep,
                      scale=1.7, shared_intermediate=shared)
    plain = _bind(moe, rng, dtype)
    h = _rounded(rng.standard_normal((T, hidden)), dtype)
    mlp = {"router": {"experts": experts, "identity": identity, "top": top, "scale": 1.7,
                      "groups": {"count": groups, "keep": keep} if groups > 1 else None}, "shared": {"ff": shared} if shared else None}
    t = pz.part(plain, "f.")
    want = pz.mixture(h, t, mlp)
    got = _np(moe.forward(None, torch.tensor(h, dtype=DT[dtype], device=DEV)))
    # rows whose choice hangs on the last bits of two scores are left out (none, or one in some hundreds)
    chosen, _ = pz.route(h, t["router"], t["correction"], mlp["router"])
    got_c, _ = K.moe_router(torch.tensor(h, dtype=DT[dtype], device=DEV), moe.router_w, moe.correction, groups, keep, top, 1.7)
    same = np.array([got_c[i].tolist() == chosen[i].tolist() for i in range(T)])
    assert same.sum() >= T - max(1, T // 50)
    assert np.abs(got - want)[same].max() <= PART_TOL[dtype] * max(1.0, np.abs(want).max())
    again = _np(moe.forward(None, torch.tensor(h, dtype=DT[dtype], device=DEV)))
    assert np.array_equal(got, again)                                         # a row's sums do not depend on its place in a segment
    if identity:                                                              # the outputs without matrices carry weight here
        assert np.abs(_identity_share(h, t, mlp)).max() > 100 * PART_TOL["float32"] * max(1.0, np.abs(want).max())
    with pytest.raises(ValueError):
        P.RoutedMoE(prefix="f.", hidden=hidden, n_experts=experts, identity=identity, top=experts + identity + 1, intermediate=ff)


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", list(zc.ALL))
def test_a_whole_prompt_then_the_rest_token_by_token(name, dtype):
    toks = H.tokens(name, 150, 1)
    want = H.plain_logits(name, toks, dtype=dtype)
    eng = H.engine(name, dtype)
    s = eng.alloc_slot()
    got = [_np(_run(eng, s, toks, 0, 100))]
    for t in range(100, 150):                                   # over the border of the second page
        got.append(_np(_run(eng, s, toks, t, t + 1)))
    H.close(np.concatenate(got), want, dtype, f"{name} prompt and decoding")


@pytest.mark.parametrize("name", list(zc.ALL))
def test_the_residual_stream_after_every_layer(name):
    toks = H.tokens(name, 40, 6)
    cfg, w = H.plain(name)
    want = []
    pz.forward(cfg, w, list(toks), want)
    eng = H.engine(name, "float32", use_graphs=False)
    got = []
    for blk in eng.model.layers:
        def wrapped(ctx, x, pending, caches, _o=blk.forward, **kw):
            x, p = _o(ctx, x, pending, caches, **kw)
            got.append(_np(x))
            return x, p
        blk.forward = wrapped
    _run(eng, eng.alloc_slot(), toks, 0, 40)
    assert len(got) == len(want) == len(cfg["layers"])
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.abs(g - w_).max() <= 5e-5 * np.abs(w_).max(), f"layer {i}"


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["zas_a", "zas_b", "zas_c"])
def test_the_first_tokens_one_by_one_and_portions_down_to_two_tokens(name, dtype):
    toks = H.tokens(name, 140, 2)
    want = H.plain_logits(name, toks, dtype=dtype)
    eng = H.engine(name, dtype, n_slots=2)
    a, b = eng.alloc_slot(), eng.alloc_slot()
    one = np.concatenate([_np(_run(eng, a, toks, t, t + 1)) for t in range(70)])          # from the very first token on
    H.close(one, want[:70], dtype, "token by token from the start")
    cuts, at, got = [2, 3, 59, 1, 2, 64, 7, 2], 0, []
    for c in cuts:
        got.append(_np(_run(eng, b, toks, at, at + c)))
        at += c
    H.close(np.concatenate(got), want, dtype, "portions")
    if dtype == "float32":                                      # in 32-bit a row's arithmetic hardly depends on the cut
        assert np.abs(np.concatenate(got)[:70] - one).max() <= 5e-5 * np.abs(want).max()


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["zas_a", "zas_c"])
def test_unequal_batches_against_each_alone_with_slots_and_pages_used_again(name, dtype):
    eng = H.engine(name, dtype, max_tokens=448, n_slots=3)              # 7 pages: the second batch needs the first one's
    for turn, lens in enumerate([(130, 9, 70), (200, 3, 66)]):
        seqs = [H.tokens(name, n + 6, 10 * turn + i) for i, n in enumerate(lens)]
        slots = [eng.alloc_slot() for _ in seqs]
        assert slots == [0, 1, 2]
        got = [[] for _ in seqs]
        out = _np(eng.step([(s, list(t[:n])) for s, t, n in zip(slots, seqs, lens)], want="all"))
        at = 0
        for i, n in enumerate(lens):
            got[i].append(out[at:at + n])
            at += n
        live = [0, 1, 2]
        for step in range(6):
            if step == 3:                                       # the shortest request ends earlier
                eng.free_slot(slots[1])
                live = [0, 2]
            out = _np(eng.step([(slots[i], [seqs[i][lens[i] + step]]) for i in live], want="all"))
            for j, i in enumerate(live):
                got[i].append(out[j:j + 1])
        for i in live:
            eng.free_slot(slots[i])
        for i, t in enumerate(seqs):
            g = np.concatenate(got[i])
            H.close(g, H.plain_logits(name, t, dtype=dtype)[:len(g)], dtype, f"{name} batch {turn} sequence {i}")
    assert eng.cache.free_pages() == [7] * len(eng.cache.groups)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["zas_b", "zas_c"])
def test_long_decoding_replayed_and_launched(name, dtype):
    toks = H.tokens(name, 210, 3)
    want = H.plain_logits(name, toks, dtype=dtype)
    outs = {}
    for graphs in (True, False):
        eng = H.engine(name, dtype, use_graphs=graphs)
        assert (eng.graphs is not None) == graphs
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 5))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(5, 210)]
        outs[graphs] = np.concatenate(got)
        H.close(outs[graphs], want, dtype, f"long decoding, graphs {graphs}")
    assert np.array_equal(outs[True], outs[False])              # a replayed step is the launched step


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_shared_expert_on_a_second_stream_changes_no_bit(dtype, monkeypatch):
    """Steps of few rows queue the shared expert beside the router and the chosen experts; with everything on one
    stream the same kernels run one after the other.  Unequal batches, prompts of few rows and single tokens, replayed
    and launched."""
    name = "zas_a"
    seqs = [H.tokens(name, 40, 30 + i) for i in range(3)]
    outs = {}
    monkeypatch.setattr(P.RoutedMoE, "side_bytes", 0)          # (a toy model's shared expert is too small to be worth a stream)
    for rows in (64, 0):
        monkeypatch.setattr(P.RoutedMoE, "side_rows", rows)
        for graphs in (True, False):
            eng = H.engine(name, dtype, use_graphs=graphs)
            slots = [eng.alloc_slot() for _ in seqs]
            got = [_np(eng.step([(s, list(t[:n])) for s, t, n in zip(slots, seqs, (20, 3, 9))], want="all"))]
            for step in range(12):
                got.append(_np(eng.step([(s, [t[n + step]]) for s, t, n in zip(slots, seqs, (20, 3, 9))], want="all")))
            outs[(rows, graphs)] = np.concatenate(got)
    first = outs[(64, True)]
    assert all(np.array_equal(first, o) for o in outs.values())
    want = np.concatenate([H.plain_logits(name, t, dtype=dtype)[:n] for t, n in zip(seqs, (20, 3, 9))])
    H.close(first[:32], want, dtype, "two streams")


def test_far_keys_the_sinks_another_layers_keys_and_the_outputs_without_matrices_decide_and_are_there():
    """On a sharpened model the logits of late positions depend on keys hundreds of positions back, on the sinks,
    on whose keys a reading layer takes and on the experts that return their input, by many times the bound; the
    engine agrees with the plain implementation that has them all."""
    name, dtype = "zas_c", "float32"
    cfg, w = H.plain(name)
    toks = H.tokens(name, 420, 4)
    want = H.plain_logits(name, toks)
    softmax, attend, mix = pz.causal_softmax, pz.attention, pz.mixture
    try:
        def without_far_keys(scores, sink=None, first=0):
            p = softmax(scores, sink, first)
            if scores.shape[0] == 420:                          # the first page, for the late queries
                cut = scores.copy(); cut[330:, :64] = -1e9
                p[330:] = softmax(cut, sink, first)[330:]
            return p
        pz.causal_softmax = without_far_keys
        no_far = pz.forward(cfg, w, list(toks))
        pz.causal_softmax = lambda scores, sink=None, first=0: softmax(scores, None if sink is None else -1e9, first)
        no_sink = pz.forward(cfg, w, list(toks))
        pz.causal_softmax = softmax
        def keys_of_their_own(h, t, m, eps, pos, keys_values=None):
            if keys_values is None:
                return attend(h, t, m, eps, pos)
            return attend(h, dict(t, k=w["l1.mix.k"], v=w["l1.mix.v"], **{"k.norm": w["l1.mix.k.norm"]}), m, eps, pos)
        pz.attention = keys_of_their_own
        own_keys = pz.forward(cfg, w, list(toks))               # the readers make keys of their own input with the owner's matrices
        pz.attention = attend
        pz.mixture = lambda h, t, mlp: mix(h, t, mlp) - _identity_share(h, t, mlp)
        no_identity = pz.forward(cfg, w, list(toks))
    finally:
        pz.causal_softmax, pz.attention, pz.mixture = softmax, attend, mix
    assert H.distance(no_far[330:], want[330:]) > 20 * H.TOL[dtype]
    for other in (no_sink, own_keys, no_identity):
        assert H.distance(other, want) > 20 * H.TOL[dtype]
    for dt in H.DTYPES:
        eng = H.engine(name, dt)
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 400))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(400, 420)]
        H.close(np.concatenate(got), H.plain_logits(name, toks, dtype=dt), dt, "far keys, sinks, read keys, outputs without matrices")


def _identity_share(h, t, mlp):
    """What the outputs without matrices add to a mixture's result."""
    r = mlp["router"]
    chosen, weights = pz.route(h, t["router"], t["correction"], r)
    out = np.zeros_like(np.asarray(h, dtype=np.float64))
    for row in range(h.shape[0]):
        for e, w_ in zip(chosen[row], weights[row]):
            if e >= r["experts"]:
                out[row] += w_ * h[row]
    return out


def test_greedy_generation_through_the_entry_point():
    name = "zas_a"
    cfg, w = H.plain(name)
    prompts = [list(H.tokens(name, 9, 7)), list(H.tokens(name, 30, 8)), list(H.tokens(name, 2, 9))]
    llm = L.Llogos(H.folder(name), dtype="float32", max_context=128, max_batch=2)        # three requests, two at a time
    out = llm.generate(prompts, L.GenerationParams.greedy(max_tokens=10, stop_tokens=()))
    for p, got in zip(prompts, out.tokens):
        assert got == pz.generate_greedy(cfg, w, p, 10)
    assert out.finish_reasons == ["length"] * 3


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_trace_runner_on_a_model_of_the_design(tmp_path, dtype):
    name = "zas_a"
    vocab = zc.ALL[name]["vocab"]
    a, b = H.tokens(name, 75, 11), H.tokens(name, 12, 12)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 63, 64, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for i in range(3):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [a[70 + i]], "want": [0]}, {"id": "b", "tokens": [b[9 + i]], "want": [0]}],
                      "end": ["b"] if i == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": list(a[73:75]), "want": [1]}], "end": ["a"]})
    out = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", H.folder(name, dtype=dtype), "--dtype", dtype, "--out", out,
           "--max-tokens", "192"]
    p = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l] == [f"done {i}" for i in range(5)]
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, vocab)
    pa, pb = H.plain_logits(name, a, dtype=dtype), H.plain_logits(name, b, dtype=dtype)
    H.close(read(0), np.concatenate([pa[[0, 63, 64, 69]], pb[8:9]]), dtype, "step 0")
    for i in range(3):
        H.close(read(1 + i), np.concatenate([pa[70 + i:71 + i], pb[9 + i:10 + i]]), dtype, f"step {1 + i}")
    H.close(read(4), pa[74:75], dtype, "step 4")


def test_the_command_line_on_a_model_of_the_design(tmp_path):
    """`random` writes a model folder from a configuration file; generation from token ids prints what the
    plain loop generates; --bench prints its block."""
    name = "zas_d"
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(zc.ALL[name]))
    out = tmp_path / "model"
    run = lambda *args: subprocess.run([sys.executable, "-m", "daisi-llogos_amd", *args], capture_output=True, text=True, timeout=600, cwd=ROOT)
    p = run("random", "--config", str(cfg_file), "--output-dir", str(out), "--seed", "4")
    assert p.returncode == 0, p.stderr[-2000:]
    cfg, w = pz.load(str(out))
    prompt = list(H.tokens(name, 11, 21))
    p = run("--model", str(out), "--prompt", " ".join(map(str, prompt)), "-n", "6", "-t", "0", "--repeat-penalty", "1.0",
            "--dtype", "float32", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.split()] == pz.generate_greedy(cfg, w, prompt, 6)
    p = run("--model", str(out), "--bench", "--batch", "2", "-n", "8", "--prompt-len", "20", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "decode" in (p.stdout + p.stderr)


def _drawn(seed: int) -> dict:
    """A configuration drawn from a seed over everything the file can vary."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(len(xs)))]
    W = int(pick(40, 48, 64, 72, 96))
    layers, owners = [], {}
    for i in range(int(rng.integers(2, 6))):
        ff = pick(None, "dense", "moe", "moe")
        mlp = None
        if ff == "dense":
            mlp = zc.dense(int(pick(24, 50, 64)))
        elif ff == "moe":
            groups = int(pick(1, 2, 3))
            per = int(pick(1, 2, 3))
            identity = int(rng.integers(0, per * groups))
            keep = int(rng.integers(1, groups + 1))
            top = int(rng.integers(1, keep * per + 1))
            mlp = zc.moe(per * groups - identity, identity, top, int(pick(8, 20, 32)), float(pick(0.5, 1.0, 2.5)),
                         groups=(groups, keep) if pick(True, groups > 1) else None, shared=int(pick(0, 16, 24)))
        if pick(True, False):
            layers.append(zc.latent(int(pick(1, 2, 5)), int(pick(8, 24, 32)), int(pick(8, 16, 40)), int(pick(8, 20, 48)), float(pick(0.2, 0.4)), mlp))
            continue
        if owners and pick(True, False):
            src = int(pick(*owners))
            o = owners[src]
            heads = o["kv_heads"] * int(pick(1, 2))
            layers.append(zc.attention(heads, o["kv_heads"], o["dim"], o["vdim"], float(pick(0.2, 0.4)), o.get("rot"), kv_from=src, mlp=mlp))
            continue
        kv = int(pick(1, 2, 3))
        dim = int(pick(8, 16, 24, 32, 64))
        dims = int(pick(0, 2, dim // 2, dim))
        rotation = None
        if dims:
            rotation = zc.rot(dims, float(pick(100.0, 10000.0)), pick(None, (4.0, 32, 8.0, 1.0), (16.0, 128, 32.0, 4.0)))
        layer = zc.attention(kv * int(pick(1, 2, 4)), kv, dim, int(pick(8, 16, 40, 64)), float(pick(0.2, 0.4)), rotation, mlp=mlp)
        owners[i] = layer["mixer"]
        layers.append(layer)
    return {"architecture": "Zasidra", "vocab": int(pick(50, 131)), "width": W, "norm": {"eps": float(pick(1e-5, 1e-6))},
            "embedding": {"scale": float(pick(1.0, 3.0))}, "layers": layers, "torch_dtype": "bfloat16"}


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_from_seeds(seed, tmp_path):
    """Ragged prompts, single tokens, a sequence that ends early and a new prompt in the freed slot beside one that goes on."""
    from safetensors.torch import load_file, save_file
    cfg = _drawn(seed)
    rng = np.random.default_rng(seed)
    seqs = [[int(t) for t in rng.integers(0, cfg["vocab"], size=n)] for n in (90, 17, 70, 40)]
    for dtype in H.DTYPES:
        path = L.write_random_model(str(tmp_path / dtype), cfg, seed=seed, std=0.08)
        file = os.path.join(path, "model.safetensors")
        save_file(H.sharpen(load_file(file), H.fixed_choice(dtype)), file)
        pcfg, w = pz.load(path)
        want = [pz.forward(pcfg, w, s) for s in seqs]
        eng = L.Engine.from_folder(path, dtype=dtype, max_tokens=512, n_slots=3)
        s0, s1, s2 = eng.alloc_slot(), eng.alloc_slot(), eng.alloc_slot()
        got = [[], [], [], []]
        out = _np(eng.step([(s0, seqs[0][:66]), (s1, seqs[1][:3]), (s2, seqs[2][:64])], want="all"))
        got[0].append(out[:66]); got[1].append(out[66:69]); got[2].append(out[69:])
        for step in range(6):
            out = _np(eng.step([(s0, [seqs[0][66 + step]]), (s1, [seqs[1][3 + step]]), (s2, [seqs[2][64 + step]])], want="all"))
            for i in range(3):
                got[i].append(out[i:i + 1])
        eng.free_slot(s1)
        s3 = eng.alloc_slot()
        assert s3 == s1
        out = _np(eng.step([(s0, seqs[0][72:90]), (s3, seqs[3][:40])], want="all"))      # a continued prompt beside a new one in the freed slot
        got[0].append(out[:18]); got[3].append(out[18:])
        for i, n in ((0, 90), (1, 9), (2, 70), (3, 40)):
            H.close(np.concatenate(got[i]), want[i][:n], dtype, f"seed {seed} sequence {i}")
