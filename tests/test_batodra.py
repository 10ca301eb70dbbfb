"""The Batodra design without a GPU: the configuration reader, the model's description (tensors, runs,
cache units), the plain implementation's mechanisms against numbers worked by hand or against
themselves continued from a carried state, and random models written and read back."""
import copy
import importlib
import math

import numpy as np
import pytest

import batodra_configs as bc
import plain_batodra as pb

L = importlib.import_module("daisi-llogos_amd")
registry = importlib.import_module("daisi-llogos_amd.config.registry")
model_mod = importlib.import_module("daisi-llogos_amd.models.model")
config_mod = importlib.import_module("daisi-llogos_amd.config.model_config")
rope = importlib.import_module("daisi-llogos_amd.parts.rope")


def _model(cfg, shapes=None):
    arch = registry.architecture_of(cfg)
    typed = arch.read_config(cfg, shapes) if shapes is not None else arch.read_config(cfg)
    return typed, model_mod.Model(arch.model_spec(typed))


def test_the_reader_takes_every_size_and_constant_from_the_file():
    typed, _ = _model(bc.BAT_A)
    assert (typed.vocab, typed.width, typed.norm_eps, typed.alpha) == (157, 80, 1e-5, 1.7)
    assert [l.type for l in typed.layers] == ["attention_2", "rglru", "attention", "rglru", "attention_2", "attention"]
    assert [l.weights_of for l in typed.layers] == [None, None, None, 1, 0, 2]
    w = typed.layers[0].mixer
    assert (w.heads, w.kv_heads, w.dim, w.vdim, w.scale, w.window, w.keep_first) == (6, 2, 24, 40, 1.0, 7, 3)
    assert (w.rot.base, w.rot.dims, w.rot.scaling) == (10000.0, 16, (4.0, 32.0, 8.0, 1.0))
    r = typed.layers[1].mixer
    assert (r.width, r.blocks, r.conv) == (96, 3, 3) and typed.layers[1].ff == 0 and typed.layers[0].ff == 48
    d = typed.layers[2].mixer
    assert (d.heads, d.kv_heads, d.dim, d.vdim, d.scale, d.diff, d.window) == (6, 2, 16, 24, 0.4, 0.3, 0)
    assert d.rot.scaling is None and typed.layers[2].ff == 112
    assert _model(bc.BAT_B)[0].alpha == 1.0


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "attention_3", "attention_3"), (("layers", 1, "mixer", "blocks"), 5, "blocks"),
    (("layers", 0, "mixer", "kv_heads"), 4, "kv_heads"), (("layers", 0, "mlp", "kind"), "moe", "moe"),
    (("layers", 3, "weights_of"), 3, "weights_of"), (("layers", 3, "weights_of"), 0, "layer 0"),
    (("layers", 2, "mixer", "rot", "dims"), 7, "dims"), (("layers", 0, "mixer", "mask", "size"), -1, "size"),
    (("norm",), None, "norm"), (("width",), "wide", "width"), (("layers", 2, "mixer", "diff"), None, "diff")])
def test_a_wrong_or_missing_key_is_named(path, value, word):
    cfg = copy.deepcopy(bc.BAT_A)
    at = cfg
    for k in path[:-1]:
        at = at[k]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(config_mod.ConfigError) as e:
        _model(cfg)
    assert word in str(e.value)


def test_a_layer_on_borrowed_tensors_is_a_second_run_with_a_cache_of_its_own():
    _, model = _model(bc.BAT_A)
    assert [e.layer for e in model.schedule] == [0, 1, 2, 1, 0, 2] and len(model.layers) == 3
    needs = model.cache_needs()
    assert len(needs) == 6 and model.cache_reads() == [None] * 6
    kv, st = needs[0]
    assert (kv.n_kv_heads, kv.head_dim, kv.value_dim, kv.window, kv.sinks) == (2, 32, 48, 7, 3) and st is None
    assert needs[4] == needs[0] and needs[3] == needs[1] and needs[5] == needs[2]
    kv, st = needs[1]
    assert kv is None and tuple(st.shape) == (3, 96)                          # two rows of the convolution's inputs, and S
    kv, st = needs[2]
    assert (kv.n_kv_heads, kv.head_dim, kv.value_dim, kv.window) == (2, 32, 32, 0)      # both maps' keys side by side; values of 24 in rows of 32
    names = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert names["embed"] == (157, 80) and names["head"] == (157, 80) and names["final.norm"] == (80,)
    assert names["l0.mix.q"] == (144, 80) and names["l0.mix.k"] == (48, 80) and names["l0.mix.v"] == (80, 80) and names["l0.mix.o"] == (80, 240)
    assert names["l1.mix.y"] == (96, 80) and names["l1.mix.x.b"] == (96,) and names["l1.mix.conv"] == (96, 3) and names["l1.mix.conv.b"] == (96,)
    assert names["l1.mix.ra"] == (3, 32, 32) and names["l1.mix.ri.b"] == (3, 32) and names["l1.mix.lam"] == (96,) and names["l1.mix.o"] == (80, 96)
    assert names["l2.mix.q"] == (192, 80) and names["l2.mix.k"] == (64, 80) and names["l2.mix.v"] == (48, 80) and names["l2.mix.o"] == (80, 144)
    assert names["l2.mix.q.norm"] == (16,) and names["l2.mix.lk2"] == (16,) and names["l2.mlp.up"] == (112, 80) and names["l2.mlp.down"] == (80, 112)
    assert "l1.norm2" not in names and "l0.norm2" in names and "l1.norm1" in names
    assert not any(n.startswith(("l3.", "l4.", "l5.", "l1.mlp")) for n in names)
    assert "l0.mix.q.norm" not in names


def test_a_second_norm_without_a_feed_forward_is_taken_from_the_tensors():
    typed, model = _model(bc.BAT_A, shapes={"l1.norm2": (80,)})
    assert typed.layers[1].second_norm and typed.layers[3].second_norm and "l1.norm2" in {s.name for s in model.tensor_specs()}


def test_a_random_model_is_written_and_read_back(tmp_path):
    path = L.write_random_model(str(tmp_path / "m"), bc.BAT_C, seed=3)
    cfg, w = pb.load_folder(path)
    assert cfg == bc.BAT_C
    logits = pb.forward(cfg, w, [1, 5, 66, 0, 5])
    assert logits.shape == (5, 67) and np.isfinite(logits).all()
    again = L.write_random_model(str(tmp_path / "n"), bc.BAT_C, seed=3)
    assert all(np.array_equal(w[k], v) for k, v in pb.load_folder(again)[1].items())


def test_the_norm_behind_the_scaled_sum_by_hand():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    assert np.allclose(pb.rms_norm(x, np.array([1.0, 2.0, 1.0, 0.5]), 0.5), x / math.sqrt(12.5 + 0.5) * [1.0, 2.0, 1.0, 0.5])
    assert np.allclose(pb.unit_rows(np.array([3.0, 4.0]), 0.0), [3.0 / math.sqrt(12.5), 4.0 / math.sqrt(12.5)])
    assert np.allclose(pb.relu_squared(np.array([-1.0, 0.5])), [0.0, 0.25])
    assert np.isclose(pb.gelu_tanh(np.array([1.0]))[0], 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715)))


def test_the_convolution_continues_from_the_rows_before():
    rng = np.random.default_rng(0)
    u, w, b = rng.standard_normal((9, 4)), rng.standard_normal((4, 3)), rng.standard_normal(4)
    whole = pb.time_convolution(u, w, b)
    assert np.allclose(whole[0], b + w[:, 2] * u[0]) and np.allclose(whole[1], b + w[:, 1] * u[0] + w[:, 2] * u[1])
    assert np.allclose(pb.time_convolution(u[5:], w, b, before=u[3:5]), whole[5:])
    assert np.allclose(pb.time_convolution(u, w[:, -1:], b), b + u * w[:, -1])      # one tap: a factor a channel


def test_the_recurrence_by_hand_and_continued():
    lam = np.array([0.0])
    sp = math.log(2.0)
    u, r, i = np.array([[2.0], [1.0]]), np.array([[0.5], [1.0]]), np.array([[1.0], [0.25]])
    out, last = pb.gated_recurrence(u, r, i, lam)
    a0, a1 = math.exp(-8 * 0.5 * sp), math.exp(-8 * sp)
    s0 = math.sqrt(1 - a0 * a0) * 2.0                                        # from S = 0: the first token has no special case
    s1 = a1 * s0 + math.sqrt(1 - a1 * a1) * 0.25
    assert np.allclose(out[:, 0], [s0, s1]) and np.isclose(last[0], s1)
    again, _ = pb.gated_recurrence(u[1:], r[1:], i[1:], lam, state=np.array([s0]))
    assert np.isclose(again[0, 0], s1)
    blocks = pb.block_products(np.array([[1.0, 2.0, 3.0, 4.0]]), np.array([[[1.0, 0.0], [1.0, 1.0]], [[0.0, 2.0], [1.0, -1.0]]]),
                               np.array([[0.5, 0.0], [0.0, 1.0]]))
    assert np.allclose(blocks, [[1.5, 3.0, 8.0, 0.0]])


def test_the_recurrent_mixer_continues_from_its_carry():
    path_cfg = bc.BAT_C
    rng = np.random.default_rng(2)
    C, hidden, taps = 48, 40, 2
    w = {"m.y": rng.standard_normal((C, hidden)), "m.y.b": rng.standard_normal(C), "m.x": rng.standard_normal((C, hidden)),
         "m.x.b": rng.standard_normal(C), "m.conv": rng.standard_normal((C, taps)), "m.conv.b": rng.standard_normal(C),
         "m.ra": rng.standard_normal((2, 24, 24)), "m.ra.b": rng.standard_normal((2, 24)), "m.ri": rng.standard_normal((2, 24, 24)),
         "m.ri.b": rng.standard_normal((2, 24)), "m.lam": rng.standard_normal(C), "m.o": rng.standard_normal((hidden, C))}
    h = rng.standard_normal((12, hidden))
    whole = pb.rglru_mixer({"conv": taps}, w, "m.", h)
    carry, got = {}, []
    for lo, hi in ((0, 1), (1, 2), (2, 7), (7, 12)):
        got.append(pb.rglru_mixer({"conv": taps}, w, "m.", h[lo:hi], carry))
    assert np.allclose(np.concatenate(got), whole) and path_cfg["layers"][2]["mixer"]["conv"] == taps


def test_the_rotation_and_its_stretched_frequencies():
    f, amp = pb.rotary_frequencies(4, 100.0)
    assert np.allclose(f, [1.0, 0.1]) and amp == 1.0
    x = np.array([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]])
    out = pb.rotate(x, [2], 4, f)
    c0, s0, c1, s1 = math.cos(2.0), math.sin(2.0), math.cos(0.2), math.sin(0.2)
    assert np.allclose(out[0, 0], [1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1, 5.0, 6.0])
    scaling = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}
    f, amp = pb.rotary_frequencies(16, 10000.0, scaling)
    base = np.array([10000.0 ** (-2.0 * i / 16) for i in range(8)])
    turns = lambda t: 16 * math.log(32 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(turns(8.0)), 0), min(math.ceil(turns(1.0)), 15)
    ramp = np.clip((np.arange(8) - lo) / max(hi - lo, 0.001), 0, 1)
    assert np.allclose(f, base / 4.0 * ramp + base * (1 - ramp)) and np.isclose(amp, 0.1 * math.log(4.0) + 1.0)
    assert f[0] == base[0] and np.isclose(f[-1], base[-1] / 4.0)
    # the library's own table of frequencies holds the same numbers
    mine = rope.Rotary(24, 16, 10000.0, scaling=dict(scaling, type="yarn"))
    assert np.allclose(mine.freqs, f, rtol=1e-12) and np.isclose(mine.amplitude, amp)


def test_the_window_keeps_the_first_tokens():
    ok = pb.visible(np.arange(8), 3, 2)
    assert ok[7].tolist() == [True, True, False, False, False, True, True, True]
    assert ok[3].tolist() == [True, True, True, True, False, False, False, False]
    assert ok[4].tolist() == [True, True, True, True, True, False, False, False]
    assert pb.visible(np.arange(5))[4].all() and not pb.visible(np.arange(5))[0, 1:].any()
    assert pb.visible(np.arange(8), 3, 0)[7].tolist() == [False] * 5 + [True] * 3


def test_differential_attention_by_hand():
    assert np.isclose(pb.difference_weight([1.0, 0.0], [0.5, 3.0], [0.0, 2.0], [1.0, -1.0], 0.25), math.exp(0.5) - math.exp(-2.0) + 0.25)
    # one head of one dimension a map, two tokens, no rotation, identity-like weights
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "diff": 0.5, "rot": {"dims": 0, "base": 10.0}}
    w = {"m.q": np.eye(4, 3), "m.k": np.eye(4, 3)[::-1].copy(), "m.v": np.array([[1.0, 0.0, 0.0], [0.0, 1.0, 1.0]]), "m.q.norm": np.ones(2),
         "m.k.norm": np.ones(2), "m.lq1": np.zeros(2), "m.lk1": np.zeros(2), "m.lq2": np.zeros(2), "m.lk2": np.zeros(2), "m.o": np.eye(2)}
    h = np.array([[1.0, 2.0, 0.5], [0.0, 1.0, 3.0]])
    out = pb.differential_attention(m, w, "m.", h, np.arange(2), 0.0)
    q, k, v = h @ w["m.q"].T, h @ w["m.k"].T, h @ w["m.v"].T
    unit = lambda x: x / np.sqrt((x * x).mean())
    maps = []
    for lo in (0, 2):
        s = np.array([unit(q[1, lo:lo + 2]) @ unit(k[j, lo:lo + 2]) for j in range(2)])
        p = np.exp(s) / np.exp(s).sum()
        maps.append(p @ v)
    o = maps[0] - 0.5 * maps[1]                                              # lam = e^0 - e^0 + diff
    assert np.allclose(out[1], unit(o) * 0.5) and np.allclose(out[0], unit(v[0] - 0.5 * v[0]) * 0.5)


def test_the_model_runs_borrowed_layers_with_the_owners_tensors():
    cfg, w = pb.load_folder(L.write_random_model(__import__("tempfile").mkdtemp(), bc.BAT_A, seed=1, std=0.1))
    toks = [3, 9, 150, 2, 77, 4, 4, 100, 31, 8, 15, 60]
    streams = []
    logits = pb.forward(cfg, w, toks, streams=streams)
    assert len(streams) == 6 and logits.shape == (12, 157)
    own = copy.deepcopy(cfg)
    for i, layer in enumerate(own["layers"]):                # the same model with every borrower's tensors written out
        src = layer.pop("weights_of", None)
        if src is not None:
            for k in [k for k in w if k.startswith(f"l{src}.")]:
                w[f"l{i}." + k.split(".", 1)[1]] = w[k]
    assert np.allclose(pb.forward(own, w, toks), logits)
    assert pb.generate_greedy(cfg, w, toks[:4], 3) == pb.generate_greedy(own, w, toks[:4], 3)
