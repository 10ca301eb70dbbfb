"""The Zasidra design without a GPU: the configuration reader, the model's description (tensors, runs,
cache units), the plain implementation's mechanisms against numbers worked by hand, and random models
written and read back."""
import copy
import importlib
import math

import numpy as np
import pytest

import plain_zasidra as pz
import zasidra_configs as zc

L = importlib.import_module("daisi-llogos_amd")
registry = importlib.import_module("daisi-llogos_amd.config.registry")
model_mod = importlib.import_module("daisi-llogos_amd.models.model")
config_mod = importlib.import_module("daisi-llogos_amd.config.model_config")
rope = importlib.import_module("daisi-llogos_amd.parts.rope")


def _model(cfg):
    arch = registry.architecture_of(cfg)
    return arch.read_config(cfg), model_mod.Model(arch.model_spec(arch.read_config(cfg)))


def test_the_reader_takes_every_size_and_constant_from_the_file():
    typed, _ = _model(zc.ZAS_A)
    assert (typed.vocab, typed.width, typed.norm_eps, typed.embedding_scale) == (199, 96, 1e-5, 2.5)
    assert [l.type for l in typed.layers] == ["attention", "latent_attention", "attention", "latent_attention"]
    m = typed.layers[0].mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.kv_from) == (4, 2, 32, 48, 0.3, None)
    assert (m.rot.dims, m.rot.base, m.rot.scaling) == (16, 10000.0, (8.0, 64.0, 16.0, 2.0))
    assert typed.layers[2].mixer.kv_from == 0 and typed.layers[2].mlp is None
    m = typed.layers[3].mixer
    assert (m.heads, m.dim, m.vdim, m.kv_rank, m.scale) == (5, 16, 8, 20, 0.4)
    f = typed.layers[0].mlp
    assert (f.kind, f.ff, f.shared_ff) == ("moe", 40, 24)
    r = f.router
    assert (r.experts, r.identity, r.outputs, r.top, r.scale, r.groups, r.keep) == (6, 2, 8, 3, 1.7, 4, 2)
    assert (typed.layers[1].mlp.kind, typed.layers[1].mlp.ff) == ("dense", 136)
    r = typed.layers[3].mlp.router
    assert (r.identity, r.groups, r.keep) == (0, 1, 1)
    typed, _ = _model(zc.ZAS_D)
    assert typed.embedding_scale == 1.0
    assert _model(zc.ZAS_B)[0].layers[3].mixer.rot is None


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "attention_9", "attention_9"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
    (("layers", 2, "mixer", "kv_from"), 1, "kv_from"), (("layers", 2, "mixer", "kv_from"), 2, "kv_from"),
    (("layers", 2, "mixer", "dim"), 16, "kv_from"), (("layers", 0, "mixer", "rot", "dims"), 7, "dims"),
    (("layers", 0, "mixer", "rot", "scaling", "slow"), None, "slow"), (("layers", 1, "mixer", "kv_rank"), None, "kv_rank"),
    (("layers", 0, "mlp", "kind"), "sparse", "sparse"), (("layers", 0, "mlp", "router", "top"), 9, "top"),
    (("layers", 0, "mlp", "router", "groups", "count"), 3, "groups"), (("layers", 0, "mlp", "router", "groups", "keep"), 1, "kept"),
    (("layers", 1, "mlp", "ff"), 0, "ff"), (("norm",), None, "norm"), (("width",), "wide", "width")])
def test_a_wrong_or_missing_key_is_named(path, value, word):
    cfg = copy.deepcopy(zc.ZAS_A)
    at = cfg
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(config_mod.ConfigError) as e:
        _model(cfg)
    assert word in str(e.value)


def test_a_reader_of_a_reader_is_refused():
    cfg = copy.deepcopy(zc.ZAS_C)
    cfg["layers"][5]["mixer"]["kv_from"] = 3
    with pytest.raises(config_mod.ConfigError) as e:
        _model(cfg)
    assert "kv_from" in str(e.value)


def test_the_description_gives_readers_their_owners_cache_and_no_key_tensors():
    _, model = _model(zc.ZAS_C)
    assert [(e.layer, e.cache_of) for e in model.schedule] == [(0, None), (1, None), (2, None), (3, 1), (4, None), (5, 1)]
    needs, reads = model.cache_needs(), model.cache_reads()
    assert reads == [None, None, None, 1, None, 1]
    assert needs[3] == (None, None) and needs[5] == (None, None)
    kv = needs[1][0]
    assert (kv.n_kv_heads, kv.head_dim, kv.value_dim) == (2, 64, 128)
    kv = needs[2][0]
    assert (kv.n_kv_heads, kv.head_dim, kv.value_dim) == (1, 128, 64)
    assert (needs[0][0].n_kv_heads, needs[0][0].head_dim) == (1, 64) and needs[4][0].head_dim == 128     # one latent row a token
    assert all(state is None for _, state in needs)
    names = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert names["l1.mix.k"] == (128, 128) and names["l1.mix.v"] == (256, 128) and names["l1.mix.k.norm"] == (128,)
    assert names["l1.mix.q.norm"] == (256,) and names["l1.mix.sink"] == (4,) and names["l1.mix.o"] == (128, 512)
    for i in (3, 5):
        assert f"l{i}.mix.q" in names and f"l{i}.mix.q.norm" in names and f"l{i}.mix.sink" in names and f"l{i}.mix.o" in names
        assert not any(n.startswith((f"l{i}.mix.k", f"l{i}.mix.v")) for n in names)
    assert names["l0.mix.q"] == (256, 128) and names["l0.mix.dkv"] == (64, 128) and names["l0.mix.dkv.norm"] == (64,)
    assert names["l0.mix.uk"] == (256, 64) and names["l0.mix.uv"] == (256, 64) and names["l0.mix.g"] == (4, 128)
    assert names["l1.mlp.router"] == (12, 128) and names["l1.mlp.correction"] == (12,)
    assert names["l1.mlp.e7.gate"] == (64, 128) and names["l1.mlp.e7.down"] == (128, 64) and "l1.mlp.e8.gate" not in names
    assert names["l1.mlp.shared.up"] == (32, 128) and "l2.mlp.shared.up" not in names
    assert names["l0.mlp.gate"] == (96, 128) and "l4.norm2" not in names and names["l4.norm1"] == (128,)
    assert names["embed"] == (190, 128) and names["head"] == (190, 128) and names["final.norm"] == (128,)
    assert model.graph_safe


def test_widths_that_are_no_multiple_of_the_pages_step_get_rows_that_are():
    _, model = _model(zc.ZAS_B)
    needs = model.cache_needs()
    assert needs[0][0].head_dim == 32                          # a latent of 24
    assert (needs[1][0].head_dim, needs[1][0].value_dim) == (32, 48)
    assert (needs[3][0].head_dim, needs[3][0].value_dim) == (16, 16)


def test_random_models_are_written_and_read_back(tmp_path):
    for name, cfg in zc.ALL.items():
        path = L.write_random_model(str(tmp_path / name), cfg, seed=3)
        got_cfg, tensors = pz.load(path)
        assert got_cfg == cfg
        _, model = _model(cfg)
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == {k: v.shape for k, v in tensors.items()}
        logits = pz.forward(got_cfg, tensors, [1, 2, 3, 4, 5])
        assert logits.shape == (5, cfg["vocab"]) and np.isfinite(logits).all()


# ---------------------------------------------------------------------------
# the plain implementation's mechanisms against numbers worked by hand
# ---------------------------------------------------------------------------
def test_the_norm_with_its_weight_stored_around_zero():
    x = np.array([[3.0, -4.0]])
    got = pz.offset_norm(x, np.array([0.5, -0.25]), 0.5)
    rms = math.sqrt(12.5 + 0.5)
    assert np.allclose(got, [[3.0 / rms * 1.5, -4.0 / rms * 0.75]])
    assert np.allclose(pz.plain_norm(x, np.array([0.5, -0.25]), 0.5), [[3.0 / rms * 0.5, 4.0 / rms * 0.25]])


def test_stretched_frequencies_by_hand_and_against_the_librarys_table():
    # 8 rotated dimensions, base 100: f_i = 100^(-i/4) = 1, 0.316.., 0.1, 0.0316..
    # pair(t) = 8 ln(40 / (2 pi t)) / (2 ln 100): pair(4) = 0.4037.., pair(0.5) = 2.2098..: lo = 0, hi = 3
    f, amp = pz.rotation_frequencies(8, 100.0, {"factor": 4.0, "original": 40, "fast": 4.0, "slow": 0.5})
    base = [100.0 ** (-i / 4.0) for i in range(4)]
    ramp = [0.0, 1.0 / 3.0, 2.0 / 3.0, 1.0]
    assert np.allclose(f, [b / 4.0 * r + b * (1.0 - r) for b, r in zip(base, ramp)])
    assert math.isclose(amp, 0.1 * math.log(4.0) + 1.0)
    lib = rope.yarn_frequencies(rope.inverse_frequencies(8, 100.0), 8, 100.0, 4.0, 40.0, 4.0, 0.5)
    assert np.allclose(lib, f, rtol=1e-14) and math.isclose(rope.yarn_amplitude(4.0), amp)
    # a ramp of no length (both ends fall on pair 0 or before it) divides by 0.001 and not by nothing: pair 0 keeps its
    # frequency, every pair behind it is slowed whole
    short = {"factor": 2.0, "original": 2 * math.pi, "fast": 4.0, "slow": 2.0}
    f, _ = pz.rotation_frequencies(4, 100.0, short)
    assert np.allclose(f, [1.0, 0.1 / 2.0])
    assert np.allclose(rope.yarn_frequencies(rope.inverse_frequencies(4, 100.0), 4, 100.0, 2.0, 2 * math.pi, 4.0, 2.0), f, rtol=1e-14)
    f, amp = pz.rotation_frequencies(6, 10.0)
    assert np.allclose(f, [1.0, 10.0 ** (-1 / 3), 10.0 ** (-2 / 3)]) and amp == 1.0


def test_the_rotation_pairs_a_dimension_with_the_one_half_the_rotated_width_on():
    x = np.arange(1.0, 7.0).reshape(1, 1, 6)                   # 4 rotated dimensions of 6: pairs (0, 2) and (1, 3)
    f = np.array([math.pi / 2.0, math.pi])
    got = pz.rotate_split_halves(np.repeat(x, 2, axis=0), np.array([0, 1]), 4, f, 2.0)
    assert np.allclose(got[0, 0], [2.0, 4.0, 6.0, 8.0, 5.0, 6.0])                  # position 0: only the amplitude
    # position 1: pair (1, 3) by 90 degrees -> (-3, 1), pair (2, 4) by 180 degrees -> (-2, -4); times 2
    assert np.allclose(got[1, 0], [-6.0, -4.0, 2.0, -8.0, 5.0, 6.0])


def test_the_sink_joins_the_denominator_once_without_a_value():
    s = np.array([[0.0, 9.0], [math.log(2.0), math.log(3.0)]])
    p = pz.causal_softmax(s, sink=math.log(5.0))
    assert np.allclose(p, [[1.0 / 6.0, 0.0], [0.2, 0.3]])
    assert np.allclose(pz.causal_softmax(s), [[1.0, 0.0], [0.4, 0.6]])
    p = pz.causal_softmax(np.zeros((1, 3)), first=1)           # a query at position 1 sees keys 0 and 1
    assert np.allclose(p, [[0.5, 0.5, 0.0]])


def test_the_router_by_hand():
    # six outputs in three groups of two; logits chosen so that s = (1, 2, 3, 4, 6, 4) / 20
    z = np.log(np.array([[1.0, 2.0, 3.0, 4.0, 6.0, 4.0]]))
    w = np.eye(6)
    r = {"experts": 4, "identity": 2, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 2}}
    # without a correction: groups score 0.1, 0.2, 0.3: the first is out; the best two are outputs 4 and 3 (the lower of the equal ones)
    chosen, weights = pz.route(z, w, np.zeros(6), r)
    assert chosen.tolist() == [[4, 3]] and np.allclose(weights, [[3.0 * 0.3 / 0.5, 3.0 * 0.2 / 0.5]])
    # a correction moves the choice and not the weights: output 0 gets +1 (its group is now the best), output 4 gets -1
    # (its group's score falls to 0.2, level with the second group's, which comes first)
    c = np.array([1.0, 0.0, 0.0, 0.0, -1.0, 0.0])
    chosen, weights = pz.route(z, w, c, r)
    assert chosen.tolist() == [[0, 3]] and np.allclose(weights, [[3.0 * 0.05 / 0.25, 3.0 * 0.2 / 0.25]])
    # outputs of a group that is out are out even when every score that is left is negative
    c = np.array([0.0, 0.0, -5.0, -5.0, -9.0, -9.0])
    chosen, _ = pz.route(z, w, c, {**r, "groups": {"count": 3, "keep": 2}, "top": 3})
    assert sorted(chosen[0].tolist()) == [0, 1, 3] and chosen[0, 0] == 1
    chosen, _ = pz.route(z, w, np.zeros(6), {**r, "groups": None, "top": 6})
    assert chosen.tolist() == [[4, 3, 5, 2, 1, 0]]


def test_outputs_without_matrices_return_their_input_and_the_shared_expert_is_added():
    rng = np.random.default_rng(0)
    W, F = 6, 4
    t = {"router": np.array([[0.0] * W, [0.0] * W]), "correction": np.array([0.0, 1.0]), "shared.gate": rng.standard_normal((F, W)),
         "shared.up": rng.standard_normal((F, W)), "shared.down": rng.standard_normal((W, F)),
         "e0.gate": rng.standard_normal((F, W)), "e0.up": rng.standard_normal((F, W)), "e0.down": rng.standard_normal((W, F))}
    h = rng.standard_normal((3, W))
    mlp = {"router": {"experts": 1, "identity": 1, "top": 1, "scale": 2.0}, "shared": {"ff": F}}
    got = pz.mixture(h, t, mlp)                                # the correction picks the output without matrices: weight 0.5 / 0.5 * 2
    assert np.allclose(got, 2.0 * h + pz.gated_ff(h, t["shared.gate"], t["shared.up"], t["shared.down"]))
    t["correction"] = np.array([1.0, 0.0])
    got = pz.mixture(h, t, {**mlp, "shared": None})
    assert np.allclose(got, 2.0 * pz.gated_ff(h, t["e0.gate"], t["e0.up"], t["e0.down"]))
    z = np.array([[1.0, -2.0]])
    assert np.allclose(pz.gated_ff(z, np.array([[1.0, 0.0]]), np.array([[0.0, 1.0]]), np.array([[2.0]])),
                       [[2.0 * (1.0 / (1.0 + math.exp(-1.0))) * -2.0]])


def test_a_layer_that_reads_anothers_keys_is_the_same_as_one_that_holds_copies_of_its_tensors():
    """The reader's result with the owner's (k, v) equals attention with the owner's key and value tensors put
    under the reader's names."""
    cfg = zc.ZAS_D
    path_cfg, tensors = cfg, {}
    rng = np.random.default_rng(1)
    _, model = _model(cfg)
    for s in model.tensor_specs():
        tensors[s.name] = rng.standard_normal(s.shape) * 0.3
    h = rng.standard_normal((9, cfg["width"]))
    pos = np.arange(9)
    m = cfg["layers"][0]["mixer"]
    own = pz.part(tensors, "l0.mix.")
    _, kv = pz.attention(h, own, m, 1e-5, pos)
    reader = pz.part(tensors, "l1.mix.")
    got, _ = pz.attention(h * 2.0, reader, m, 1e-5, pos, kv)
    full = dict(reader, **{n: own[n] for n in ("k", "k.norm", "v")})
    # (the copies see the reader's input; the owner saw its own: feed the copies the owner's input through k and v alone)
    want_q = pz.attention(h * 2.0, full, m, 1e-5, pos, pz.attention_keys_values(h, full, m, 1e-5, pos))[0]
    assert np.allclose(got, want_q)
