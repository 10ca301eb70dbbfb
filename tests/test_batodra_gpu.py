"""The Batodra design on the GPU against the plain implementation: every mechanism alone (the norm behind
the scaled sum, the gated recurrence with its convolution, differential attention, window attention with
kept first tokens and unit-length queries and keys), whole prompts, prompts cut into portions,
token-by-token decoding, unequal batches with slots and pages used again, long decoding over page and
window borders, sensitivity to a far key, to the window's two edges, to the kept first tokens and to the
carried state, greedy generation through the library's entry point, and the trace runner and the command
line as programs."""
import importlib
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import batodra_configs as bc
import batodra_helpers as H
import plain_batodra as pb

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


def _bind(part, rng, dtype, scale=0.3, scaled=None, shifted=None):
    """Random tensors for a part (stored in bfloat16, as a model folder holds them); returns them as float64."""
    tensors, plain = {}, {}
    lim = {"norm": (0.7, 1.3), "taps": (-0.8, 0.8), "bonus": (-6.0, 1.0)}
    for spec in part.tensor_specs():
        if spec.kind in lim:
            t = torch.tensor(rng.uniform(*lim[spec.kind], size=spec.shape), dtype=torch.bfloat16)
        else:
            v = rng.standard_normal(spec.shape) * scale * (scaled or {}).get(spec.name, 1.0) + (shifted or {}).get(spec.name, 0.0)
            t = torch.tensor(v, dtype=torch.bfloat16)
        tensors[spec.name], plain[spec.name] = t, t.double().numpy()
    part.bind(tensors.get, P.Runtime(DEV, DT[dtype]))
    return plain


def _rebind(part, plain, dtype):
    part.bind({k: torch.tensor(v, dtype=torch.bfloat16) for k, v in plain.items()}.get, P.Runtime(DEV, DT[dtype]))


def _run(eng, slot, toks, lo, hi):
    return eng.step([(slot, list(toks[lo:hi]))], want="all")


def _pieces(mix, dtype, h, lengths, cuts, pages, slots, n_pages=9, poison=4):
    """Runs a mixer alone over sequences cut into steps; their pages lie in any order, and one page that
    belongs to nobody is full of NaN.  Returns a [n, hidden] array for each sequence."""
    spec, st = mix.kv_spec(), mix.state_spec()
    k_pool = v_pool = None
    if spec is not None:
        k_pool = torch.zeros((n_pages, spec.n_kv_heads, 64 * spec.head_dim), dtype=DT[dtype], device=DEV)
        v_pool = torch.zeros((n_pages, spec.n_kv_heads, 64 * spec.value_dim), dtype=DT[dtype], device=DEV)
        k_pool[poison] = float("nan")
        v_pool[poison] = float("nan")
    state = torch.zeros((max(slots) + 2,) + tuple(st.shape), dtype=torch.float32, device=DEV) if st is not None else None
    hidden = h[0].shape[1]
    got = [np.zeros((n, hidden)) for n in lengths]
    width = max(len(p) for p in pages.values()) if pages else 1
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(mix.rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        table = None
        if spec is not None:
            tab = np.full((len(seqs), width), -1, dtype=np.int32)
            for r, i in enumerate(seqs):
                tab[r, :len(pages[i])] = pages[i]
            table = _i32(tab)
        cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=table, state=state)
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), dtype=DT[dtype], device=DEV)
        o = _np(K.sum_parts(mix.forward(ctx, rows, cache), None, torch.float32))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    return got


LENGTHS = (150, 70, 3)
CUTS = [(60, 9, 1), (1, 1, 1), (1, 1, 1), (3, 58, 0), (1, 1, 0), (2, 0, 0), (64, 0, 0), (1, 0, 0), (17, 0, 0)]
PAGES = {0: [7, 2, 5], 1: [0, 8], 2: [3]}
SLOTS = [1, 3, 0]


def _inputs(rng, hidden, dtype, lengths=LENGTHS):
    return [np.asarray(torch.tensor(rng.standard_normal((n, hidden))).to(DT[dtype]).double()) for n in lengths]


# ---------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("width", [6, 70, 192, 1000, 5000])
@pytest.mark.parametrize("rows", ["float32", "bfloat16"])
def test_the_norm_behind_the_scaled_sum(width, rows):
    rng = np.random.default_rng(width)
    x = rng.standard_normal((11, width)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, size=width).astype(np.float32)
    for delta in (None, rng.standard_normal((11, width)).astype(np.float32), rng.standard_normal((3, 11, width)).astype(np.float32)):
        for alpha in (1.0, 2.75):
            xs = torch.tensor(x, device=DEV)
            d = None if delta is None else torch.tensor(delta, device=DEV)
            out = K.post_norm(xs, d, alpha, torch.tensor(w, device=DEV), 1e-5, DT[rows])
            total = alpha * x.astype(np.float64) + (0 if delta is None else delta.astype(np.float64).reshape(-1, 11, width).sum(0))
            want = pb.rms_norm(total, w, 1e-5)
            assert np.abs(_np(xs) - want).max() <= 1e-5 * np.abs(want).max()
            assert out.dtype == DT[rows] and np.abs(_np(out) - want).max() <= PART_TOL[rows] * np.abs(want).max()


# (hidden, channels, blocks, taps)
RECURRENT = [(56, 96, 3, 3), (64, 256, 8, 4), (40, 48, 1, 1), (48, 60, 2, 2), (32, 1024, 4, 4)]


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("segment", [0, 64, -1])
@pytest.mark.parametrize("shape", RECURRENT)
def test_the_recurrent_mixer_alone_in_pieces(shape, segment, dtype, monkeypatch):
    """Three sequences cut into steps of several sizes, with a prompt step cut into segments that run side by
    side, left to the step's own choice, or never cut.  The decays reach from a token to hundreds of tokens."""
    hidden, C, blocks, taps = shape
    monkeypatch.setattr(K, "RECURRENCE_SEGMENT", segment)
    rng = np.random.default_rng(C + taps)
    mix = P.RGLRU(prefix="m.", hidden=hidden, width=C, blocks=blocks, conv_taps=taps)
    plain = _bind(mix, rng, dtype, scaled={"m.ra": 3.0, "m.ri": 3.0})
    h = _inputs(rng, hidden, dtype)
    want = [pb.rglru_mixer({"conv": taps}, plain, "m.", x) for x in h]
    got = _pieces(mix, dtype, h, LENGTHS, CUTS, None, SLOTS)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.isfinite(g).all()
        assert np.abs(g - w_).max() <= PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"


def test_the_recurrence_carries_a_loud_token_over_hundreds_of_steps():
    """A channel whose decay is close to one keeps a loud early input: the output hundreds of tokens later
    depends on it by many times the bound; a state that was lost between steps, or the convolution's rows,
    would show."""
    hidden, C, blocks, taps = 32, 64, 2, 4
    rng = np.random.default_rng(1)
    mix = P.RGLRU(prefix="m.", hidden=hidden, width=C, blocks=blocks, conv_taps=taps)
    plain = _bind(mix, rng, "float32", shifted={"m.ra.b": -4.0})          # small r: a close to one
    n = 400
    h = rng.standard_normal((n, hidden)) * 0.5
    h[2] *= 12.0
    want = pb.rglru_mixer({"conv": taps}, plain, "m.", h)
    quiet = h.copy()
    quiet[2] /= 12.0
    assert np.abs(pb.rglru_mixer({"conv": taps}, plain, "m.", quiet)[380:] - want[380:]).max() > 100 * PART_TOL["float32"] * np.abs(want).max()
    carry = {}
    head = pb.rglru_mixer({"conv": taps}, plain, "m.", h[:300], carry)
    lost_conv = dict(carry, conv=np.zeros_like(carry["conv"]))
    assert np.abs(pb.rglru_mixer({"conv": taps}, plain, "m.", h[300:], lost_conv)[0] - want[300]).max() > 100 * PART_TOL["float32"] * np.abs(want).max()
    assert np.allclose(np.concatenate([head, pb.rglru_mixer({"conv": taps}, plain, "m.", h[300:], carry)]), want)
    for dtype in H.DTYPES:
        _rebind(mix, plain, dtype)
        got = _pieces(mix, dtype, [h], (n,), [(300,)] + [(1,)] * 98 + [(2,)], None, [2])[0]
        assert np.abs(got - want).max() <= PART_TOL[dtype] * np.abs(want).max()


# (heads, kv heads, key width of a map, value width, hidden, rotated width)
DIFFERENTIAL = [(6, 2, 16, 24, 56, 16), (2, 2, 64, 128, 64, 32), (1, 1, 8, 40, 40, 2), (4, 1, 32, 64, 48, 8), (3, 3, 24, 16, 72, 0),
                (4, 2, 64, 64, 64, 64), (8, 2, 32, 32, 64, 16), (2, 1, 128, 128, 96, 64)]


def _differential(heads, kv, d, dv, hidden, rot, diff=0.3, scale=0.5, base=100.0, window=0, keep=0):
    position = P.Rotary(d, rot, base) if rot else None
    return P.DiffAttention(prefix="m.", hidden=hidden, n_heads=heads, n_kv_heads=kv, head_dim=d, v_dim=dv, scale=scale, diff=diff,
                           position=position, eps=1e-5, window=window, sinks=keep)


def _on_the_matrix_cores(monkeypatch, d, dv):
    """Shapes that the matrix-core kernels take must run there in bfloat16."""
    if d in (32, 64, 128) and dv in (64, 128):
        check = K._check
        monkeypatch.setattr(K, "_check", lambda code, name: pytest.fail("the kernel for any shape ran") if name == "diff_attention_generic"
                            else check(code, name))


def _plain_differential(mix, plain, h, rot, base=100.0):
    m = {"heads": mix.n_heads, "kv_heads": mix.n_kv_heads, "dim": mix.head_dim, "vdim": mix.v_dim, "scale": mix.scale,
         "diff": mix.diff, "rot": {"dims": rot, "base": base}}
    return pb.differential_attention(m, plain, "m.", h, np.arange(len(h)), mix.eps)


@pytest.mark.parametrize("dtype,halves", [("float32", 0), ("bfloat16", 0), ("bfloat16", 1), ("bfloat16", 2)])
@pytest.mark.parametrize("shape", DIFFERENTIAL)
def test_differential_attention_alone_in_pieces(shape, dtype, halves, monkeypatch):
    heads, kv, d, dv, hidden, rot = shape
    monkeypatch.setattr(K, "DIFF_PREFILL_HALVES", halves)            # either form of the prompt kernel in turn
    if dtype == "bfloat16":
        _on_the_matrix_cores(monkeypatch, d, dv)
    rng = np.random.default_rng(heads * 100 + d)
    mix = _differential(*shape)
    plain = _bind(mix, rng, dtype, scaled={"m.lq1": 2.0, "m.lk2": 2.0})
    h = _inputs(rng, hidden, dtype)
    want = [_plain_differential(mix, plain, x, rot) for x in h]
    got = _pieces(mix, dtype, h, LENGTHS, CUTS, PAGES, SLOTS)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.isfinite(g).all()
        assert np.abs(g - w_).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 64, 64, 64, 64), (6, 2, 16, 24, 56, 16)])
def test_differential_attention_behind_a_window_that_keeps_the_first_tokens(shape, dtype, monkeypatch):
    """The mixer takes a window like the plain attention does (the design's own layers give it none)."""
    heads, kv, d, dv, hidden, rot = shape
    if dtype == "bfloat16":
        _on_the_matrix_cores(monkeypatch, d, dv)
    rng = np.random.default_rng(d)
    mix = _differential(*shape, window=70, keep=3)
    plain = _bind(mix, rng, dtype)
    h = _inputs(rng, hidden, dtype)
    sees = pb.visible
    monkeypatch.setattr(pb, "visible", lambda p, window=0, keep_first=0: sees(p, 70, 3))
    want = [_plain_differential(mix, plain, x, rot) for x in h]
    got = _pieces(mix, dtype, h, LENGTHS, CUTS, PAGES, SLOTS)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.abs(g - w_).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"


@pytest.mark.parametrize("dv", [48, 64])
def test_a_far_key_decides_in_each_map_of_differential_attention(dv):
    """The query matrix of one map is the key matrix with its columns reversed, and the late tokens are an early
    token reversed: their queries point at that token's key in that map alone, so it outweighs hundreds of others.
    Without that key the plain result moves by many times the bound, for either map; the kernels agree with it there."""
    heads, kv, d, hidden, rot = 4, 2, 32, 64, 8
    for which in (0, 1):
        rng = np.random.default_rng(7 + which)
        mix = _differential(heads, kv, d, dv, hidden, rot, scale=1.0, base=50000.0)
        plain = _bind(mix, rng, "float32")
        q = plain["m.q"].reshape(heads, 2, d, hidden)
        k = plain["m.k"].reshape(kv, 2, d, hidden)
        for hq in range(heads):
            q[hq, which] = k[hq // (heads // kv), which][:, ::-1]
        n = 330
        h = rng.standard_normal((n, hidden))
        h[300:] = h[5][::-1] + 0.05 * rng.standard_normal((30, hidden))
        want = _plain_differential(mix, plain, h, rot, base=50000.0)
        moved = h.copy()
        moved[5] = rng.standard_normal(hidden)
        other = _plain_differential(mix, plain, moved, rot, base=50000.0)
        assert np.abs(other[300:] - want[300:]).max() > 100 * PART_TOL["float32"] * np.abs(want).max()
        for dtype in H.DTYPES:
            _rebind(mix, plain, dtype)
            got = _pieces(mix, dtype, [h], (n,), [(257,)] + [(1,)] * 60 + [(13,)], {0: [4, 1, 0, 5, 2, 3]}, [0], n_pages=7, poison=6)[0]
            assert np.abs(got - want).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * np.abs(want).max()


# (heads, kv heads, key width, value width, hidden, rotated width, window, first tokens kept, stretched frequencies)
WINDOWED = [(6, 2, 24, 40, 56, 16, 7, 3, True), (4, 1, 64, 64, 64, 64, 33, 0, True), (2, 2, 128, 128, 64, 32, 70, 6, False),
            (1, 1, 40, 8, 40, 20, 500, 2, False), (3, 3, 16, 24, 48, 16, 5, 1, True), (8, 4, 64, 64, 64, 64, 64, 1, True),
            (4, 2, 64, 32, 32, 16, 65, 5, False), (2, 1, 96, 96, 48, 96, 1, 1, False), (2, 2, 32, 32, 32, 0, 9, 0, False)]
SCALING = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}


def _windowed(heads, kv, d, dv, hidden, rot, window, keep, stretched, scale=None):
    position = None
    if rot:
        position = P.Rotary(d, rot, 10000.0, scaling=dict(SCALING, type="yarn") if stretched else None)
    return P.Attention(prefix="m.", hidden=hidden, n_heads=heads, n_kv_heads=kv, head_dim=d, v_dim=dv, scale=scale or 4.0 / d,
                       position=position, eps=1e-5, window=window, sinks=keep, unit_qk=True, names=("q", "k", "v", "o"), suffix="")


def _plain_windowed(mix, plain, h, rot, stretched, window=None, keep=None):
    m = {"heads": mix.n_heads, "kv_heads": mix.n_kv_heads, "dim": mix.head_dim, "vdim": mix.v_dim, "scale": mix.scale,
         "rot": {"dims": rot, "base": 10000.0, "scaling": SCALING if stretched else None},
         "mask": {"size": mix.window if window is None else window, "keep_first": mix.sinks if keep is None else keep}}
    return pb.window_attention(m, plain, "m.", h, np.arange(len(h)), mix.eps)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("shape", WINDOWED)
def test_window_attention_alone_in_pieces(shape, dtype):
    heads, kv, d, dv, hidden, rot, window, keep, stretched = shape
    rng = np.random.default_rng(heads * 100 + d + window)
    mix = _windowed(*shape)
    plain = _bind(mix, rng, dtype)
    h = _inputs(rng, hidden, dtype)
    want = [_plain_windowed(mix, plain, x, rot, stretched) for x in h]
    got = _pieces(mix, dtype, h, LENGTHS, CUTS, PAGES, SLOTS)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.isfinite(g).all()
        assert np.abs(g - w_).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"


@pytest.mark.parametrize("shape", [(2, 1, 24, 40, 32, 8, 7, 3, True), (2, 2, 64, 64, 32, 64, 66, 2, False)])
def test_the_windows_edges_and_the_kept_tokens_decide(shape):
    """A window one key longer or shorter, one kept token more or fewer: the plain result moves by many times the
    bound at every late position, in prompts and in decoding; the kernels agree with the window as given."""
    heads, kv, d, dv, hidden, rot, window, keep, stretched = shape
    rng = np.random.default_rng(window)
    mix = _windowed(*shape, scale=6.0 / d)
    plain = _bind(mix, rng, "float32")
    n = 200
    h = rng.standard_normal((n, hidden))
    want = _plain_windowed(mix, plain, h, rot, stretched)
    late = slice(window + keep + 2, n)
    for dw, dk in ((1, 0), (-1, 0), (0, 1), (0, -1)):
        other = _plain_windowed(mix, plain, h, rot, stretched, window + dw, keep + dk)
        gaps = np.abs(other[late] - want[late]).max(axis=1)
        assert gaps.min() > 20 * PART_TOL["float32"] * np.abs(want).max(), (dw, dk)
    for dtype in H.DTYPES:
        _rebind(mix, plain, dtype)
        got = _pieces(mix, dtype, [h], (n,), [(100,)] + [(1,)] * 80 + [(2,)] * 10, {0: [4, 1, 0, 5]}, [0], n_pages=7, poison=6)[0]
        assert np.abs(got - want).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * np.abs(want).max()


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", list(bc.ALL))
def test_a_whole_prompt_then_the_rest_token_by_token(name, dtype):
    toks = H.tokens(name, 150, 1)
    want = H.plain_logits(name, toks)
    eng = H.engine(name, dtype)
    s = eng.alloc_slot()
    got = [_np(_run(eng, s, toks, 0, 100))]
    for t in range(100, 150):                                   # over the border of the second page
        got.append(_np(_run(eng, s, toks, t, t + 1)))
    H.close(np.concatenate(got), want, dtype, f"{name} prompt and decoding")


@pytest.mark.parametrize("name", list(bc.ALL))
def test_the_residual_stream_after_every_run_of_a_layer(name):
    toks = H.tokens(name, 40, 6)
    cfg, w = H.plain(name)
    want = []
    pb.forward(cfg, w, list(toks), streams=want)
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
        assert np.abs(g - w_).max() <= 2e-5 * np.abs(w_).max(), f"run {i}"


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", list(bc.ALL))
def test_the_first_tokens_one_by_one_and_portions_down_to_two_tokens(name, dtype):
    toks = H.tokens(name, 140, 2)
    want = H.plain_logits(name, toks)
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
@pytest.mark.parametrize("name", ["bat_a", "bat_b"])
def test_unequal_batches_against_each_alone_with_slots_and_pages_used_again(name, dtype):
    eng = H.engine(name, dtype, max_tokens=448, n_slots=3)              # 7 pages: the second batch needs the first one's
    for round_, lens in enumerate([(130, 9, 70), (200, 3, 66)]):
        seqs = [H.tokens(name, n + 6, 10 * round_ + i) for i, n in enumerate(lens)]
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
            H.close(g, H.plain_logits(name, t)[:len(g)], dtype, f"{name} round {round_} sequence {i}")
    assert eng.cache.free_pages() == [7] * len(eng.cache.groups)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["bat_a", "bat_c"])
def test_long_decoding_replayed_and_launched(name, dtype):
    toks = H.tokens(name, 210, 3)
    want = H.plain_logits(name, toks)
    outs = {}
    for graphs in (True, False):
        eng = H.engine(name, dtype, use_graphs=graphs)
        assert (eng.graphs is not None) == graphs
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 5))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(5, 210)]
        outs[graphs] = np.concatenate(got)
        H.close(outs[graphs], want, dtype, f"long decoding, graphs {graphs}")
    assert np.array_equal(outs[True], outs[False])              # a replayed step is the launched step


def test_far_keys_both_edges_the_kept_tokens_and_the_state_decide_and_are_there():
    """On a sharpened model the logits of late positions depend by many times the bound on keys hundreds of
    positions back, on the window's length to the token, on the number of kept first tokens and on the state that
    the recurrence carries; the engine agrees with the plain implementation that has them as given."""
    name, dtype = "bat_a", "float32"
    cfg, w = H.plain(name)
    toks = H.tokens(name, 420, 4)
    want = H.plain_logits(name, toks)
    sees, recur = pb.visible, pb.gated_recurrence
    try:
        others = {}
        for what, (dw, dk) in {"window + 1": (1, 0), "window - 1": (-1, 0), "kept + 1": (0, 1), "kept - 1": (0, -1)}.items():
            pb.visible = lambda p, window=0, keep_first=0: sees(p, window + dw if window else 0, keep_first + dk if window else 0)
            others[what] = pb.forward(cfg, w, list(toks))

        def without_far_keys(p, window=0, keep_first=0):
            ok = sees(p, window, keep_first)
            if not window:
                ok[330:, :64] = False                           # the first page, for the late queries
            return ok
        pb.visible = without_far_keys
        others["far keys"] = pb.forward(cfg, w, list(toks))
        pb.visible = sees

        def forgetful(u, r, i, lam, state=None):
            head, last = recur(u[:400], r[:400], i[:400], lam, state)
            tail, last = recur(u[400:], r[400:], i[400:], lam, None)         # the state is lost where the prompt ends
            return np.concatenate([head, tail]), last
        pb.gated_recurrence = forgetful
        others["state"] = pb.forward(cfg, w, list(toks))
    finally:
        pb.visible, pb.gated_recurrence = sees, recur
    for what, other in others.items():
        assert H.distance(other[400:], want[400:]) > 20 * H.TOL[dtype], what
    for dt in H.DTYPES:
        eng = H.engine(name, dt)
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 400))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(400, 420)]
        H.close(np.concatenate(got), want, dt, "far keys, edges, kept tokens and state")


def test_greedy_generation_through_the_entry_point():
    name = "bat_a"
    cfg, w = H.plain(name)
    prompts = [list(H.tokens(name, 9, 7)), list(H.tokens(name, 30, 8)), list(H.tokens(name, 2, 9))]
    llm = L.Llogos(H.folder(name), dtype="float32", max_context=128, max_batch=2)        # three requests, two at a time
    out = llm.generate(prompts, L.GenerationParams.greedy(max_tokens=10, stop_tokens=()))
    for p, got in zip(prompts, out.tokens):
        assert got == pb.generate_greedy(cfg, w, p, 10)
    assert out.finish_reasons == ["length"] * 3


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_trace_runner_on_a_model_of_the_design(tmp_path, dtype):
    name = "bat_a"
    vocab = bc.ALL[name]["vocab"]
    a, b = H.tokens(name, 75, 11), H.tokens(name, 12, 12)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 63, 64, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for i in range(3):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [a[70 + i]], "want": [0]}, {"id": "b", "tokens": [b[9 + i]], "want": [0]}],
                      "end": ["b"] if i == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": list(a[73:75]), "want": [1]}], "end": ["a"]})
    out = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", H.folder(name), "--dtype", dtype, "--out", out,
           "--max-tokens", "192"]
    p = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l] == [f"done {i}" for i in range(5)]
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, vocab)
    pa, pb_ = H.plain_logits(name, a), H.plain_logits(name, b)
    H.close(read(0), np.concatenate([pa[[0, 63, 64, 69]], pb_[8:9]]), dtype, "step 0")
    for i in range(3):
        H.close(read(1 + i), np.concatenate([pa[70 + i:71 + i], pb_[9 + i:10 + i]]), dtype, f"step {1 + i}")
    H.close(read(4), pa[74:75], dtype, "step 4")


def test_the_command_line_on_a_model_of_the_design(tmp_path):
    """`random` writes a model folder from a configuration file; generation from token ids prints what the
    plain loop generates; --bench prints its block."""
    name = "bat_c"
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(bc.ALL[name]))
    out = tmp_path / "model"
    run = lambda *args: subprocess.run([sys.executable, "-m", "daisi-llogos_amd", *args], capture_output=True, text=True, timeout=600, cwd=ROOT)
    p = run("random", "--config", str(cfg_file), "--output-dir", str(out), "--seed", "4")
    assert p.returncode == 0, p.stderr[-2000:]
    cfg, w = pb.load_folder(str(out))
    prompt = list(H.tokens(name, 11, 21))
    p = run("--model", str(out), "--prompt", " ".join(map(str, prompt)), "-n", "6", "-t", "0", "--repeat-penalty", "1.0",
            "--dtype", "float32", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.split()] == pb.generate_greedy(cfg, w, prompt, 6)
    p = run("--model", str(out), "--bench", "--batch", "2", "-n", "8", "--prompt-len", "20", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "decode" in (p.stdout + p.stderr)


# ---------------------------------------------------------------------------
# configurations drawn at random
# ---------------------------------------------------------------------------
def random_batodra_config(seed: int) -> dict:
    """Everything config.json can vary, drawn from a seed: widths and vocabularies that are no power of two, three to
    seven layers of any type in any order, some of them on an earlier layer's tensors, with or without a feed-forward;
    head sizes in steps of 8, heads and groups, values wider or narrower than keys, whole or partial rotations with
    or without stretched frequencies, windows from one key to longer than the test, none to eight kept tokens; one
    to six taps, one to eight blocks."""
    rng = np.random.default_rng(7000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]

    def rot(dim):
        dims = int(pick([dim, dim, max(2, dim // 2), max(2, (dim // 4) * 2), 2]))
        scaling = None
        if pick([True, False]):
            scaling = (float(pick([2.0, 4.0, 8.0, 32.0])), int(pick([16, 64, 512])), float(pick([4.0, 32.0])), float(pick([0.5, 1.0, 2.0])))
        return (float(pick([50.0, 1e4, 5e5])), dims, scaling)

    def layer():
        kind = pick(["rglru", "attention", "attention_2"])
        ff = pick([None, int(pick([24, 56, 96, 136, 256]))])
        if kind == "rglru":
            blocks = int(pick([1, 2, 3, 4, 8]))
            return bc.recurrent(blocks * int(pick([8, 12, 16, 32, 40, 64])), blocks, int(pick([1, 2, 3, 4, 6])), ff=ff)
        kv = int(pick([1, 2, 3, 4]))
        heads = kv * int(pick([1, 1, 2, 3, 4]))
        if kind == "attention":
            dim = int(pick([8, 16, 24, 32, 32, 64, 64, 128]))
            dv = int(pick([dim, 2 * dim, 16, 40, 64, 128]))
            return bc.differential(heads, kv, dim, dv, float(pick([dim ** -0.5, 0.3, 0.1])), float(pick([0.2, 0.5, 0.8])), rot(dim)[:2] +
                                   ((rot(dim)[2],) if pick([False, False, True]) else ()), ff=ff)
        dim = int(pick([8, 16, 24, 40, 64, 64, 96, 128]))
        dv = int(pick([dim, dim, 16, 48, 64, 128]))
        return bc.windowed(heads, kv, dim, dv, float(pick([8.0, 12.0, 4.0])) / dim, rot(dim), int(pick([1, 5, 33, 40, 64, 65, 100, 1000])),
                           int(pick([0, 0, 1, 4, 6, 8])), ff=ff)

    layers = []
    for i in range(int(pick([3, 4, 5, 6, 7]))):
        if layers and pick([True, False, False]):
            src = int(rng.integers(0, len(layers)))
            src = layers[src].get("weights_of", src)
            new = {k: v for k, v in layers[src].items()}
            new["weights_of"] = src
            layers.append(new)
        else:
            layers.append(layer())
    return {"architecture": "Batodra", "vocab": int(pick([67, 131, 256, 577, 1000])), "width": int(pick([40, 64, 72, 96, 136, 192, 256])),
            "norm": {"eps": float(pick([1e-6, 1e-5, 1e-4]))}, "postln_alpha": float(pick([1.0, 1.5, 2.5, 4.0])), "layers": layers,
            "torch_dtype": "bfloat16"}


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("seed", list(range(16)))
def test_random_configuration(seed, dtype):
    """Ragged prompts in one step, single tokens with a sequence ending early, then a continued prompt beside a new one
    in the freed slot, against the plain implementation."""
    name = f"random_{seed}"
    bc.ALL[name] = random_batodra_config(seed)
    rng = np.random.default_rng(seed)
    lens = [int(rng.integers(1, 150)) for _ in range(3)]
    seqs = [H.tokens(name, n + 8, 10 * seed + i) for i, n in enumerate(lens)]
    plain = [H.plain_logits(name, s) for s in seqs]
    eng = H.engine(name, dtype, max_tokens=64 * 12, n_slots=3)
    slots = [eng.alloc_slot() for _ in seqs]
    got = eng.step([(sl, list(s[:n])) for sl, s, n in zip(slots, seqs, lens)], want="all")
    H.close(_np(got), np.concatenate([p[:n] for p, n in zip(plain, lens)]), dtype, f"{name}: prompts")
    live = [0, 1, 2]
    for t in range(6):
        if t == 3:                                      # the second sequence ends early; its slot takes a new prompt later
            eng.free_slot(slots[1])
            live = [0, 2]
        got = eng.step([(slots[i], [seqs[i][lens[i] + t]]) for i in live], want="last")
        H.close(_np(got), np.stack([plain[i][lens[i] + t] for i in live]), dtype, f"{name}: token {t}")
    slots[1] = eng.alloc_slot()
    got = eng.step([(slots[0], list(seqs[0][lens[0] + 6:lens[0] + 8])), (slots[1], list(seqs[1][:lens[1]]))], want=[[0, 1], [lens[1] - 1]])
    want = np.stack([plain[0][lens[0] + 6], plain[0][lens[0] + 7], plain[1][lens[1] - 1]])
    H.close(_np(got), want, dtype, f"{name}: a continued prompt beside a new one")
