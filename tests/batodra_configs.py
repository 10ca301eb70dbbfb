"""Small configurations of the Batodra design for tests.  Between them every size differs from layer to
layer and from the others of its layer (query heads equal to the key/value heads, twice and three times
as many; key and value widths that differ either way; rotations over a part of a head and over all of it,
with and without the stretched frequencies; widths that are no multiple of 16), the three layer types come
in several orders, with and without a feed-forward, with and without layers that run another layer's
tensors, and the constants take values that matter within a test's length (windows of 5 and 33 tokens,
none to six first tokens kept, one to four taps, one to eight blocks) or make a mechanism trivial
(a window longer than any test, one tap, one block, a factor of one on the stream)."""


def recurrent(width, blocks, conv, ff=None, weights_of=None):
    layer = {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv},
             "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


def _rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def differential(heads, kv_heads, dim, vdim, scale, diff, rot, ff=None, weights_of=None):
    layer = {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                            "diff": diff, "rot": _rot(*rot)},
             "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


def windowed(heads, kv_heads, dim, vdim, scale, rot, window, keep_first, ff=None, weights_of=None):
    layer = {"type": "attention_2", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                              "rot": _rot(*rot), "mask": {"size": window, "keep_first": keep_first}},
             "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


BAT_A = {   # every type, then every type again on the first ones' tensors; three query heads a kv head in both attentions
    "architecture": "Batodra", "vocab": 157, "width": 80, "norm": {"eps": 1e-5}, "postln_alpha": 1.7,
    "layers": [windowed(6, 2, 24, 40, 1.0, (10000.0, 16, (4.0, 32, 8.0, 1.0)), 7, 3, ff=48),
               recurrent(96, 3, 3),
               differential(6, 2, 16, 24, 0.4, 0.3, (100.0, 16), ff=112),
               recurrent(96, 3, 3, weights_of=1),
               windowed(6, 2, 24, 40, 1.0, (10000.0, 16, (4.0, 32, 8.0, 1.0)), 7, 3, ff=48, weights_of=0),
               differential(6, 2, 16, 24, 0.4, 0.3, (100.0, 16), ff=112, weights_of=2)],
    "torch_dtype": "bfloat16",
}

BAT_B = {   # head shapes that the matrix-core kernels take; no borrowed tensors; no first tokens kept; one block; one tap
    "architecture": "Batodra", "vocab": 190, "width": 128, "norm": {"eps": 1e-6}, "postln_alpha": 1.0,
    "layers": [recurrent(256, 8, 4, ff=96),
               windowed(4, 1, 64, 64, 0.4, (500000.0, 64, (8.0, 64, 16.0, 2.0)), 33, 0, ff=64),
               differential(2, 2, 64, 128, 0.2, 0.6, (1000.0, 32), ff=160),
               recurrent(64, 1, 1),
               windowed(2, 2, 128, 128, 0.2, (10000.0, 32), 70, 6),
               differential(4, 2, 32, 64, 0.3, 0.1, (50.0, 8, (2.0, 16, 4.0, 1.0)), ff=32)],
    "torch_dtype": "bfloat16",
}

BAT_C = {   # one head; a window longer than any test; a width that is no multiple of 16; a borrower of a layer without a feed-forward
    "architecture": "Batodra", "vocab": 67, "width": 40, "norm": {"eps": 1e-5}, "postln_alpha": 3.0,
    "layers": [differential(1, 1, 8, 40, 0.7, 0.8, (20.0, 2)),
               windowed(1, 1, 40, 8, 0.6, (300.0, 20), 500, 2, ff=24),
               recurrent(48, 2, 2, ff=56),
               differential(1, 1, 8, 40, 0.7, 0.8, (20.0, 2), weights_of=0),
               windowed(3, 3, 16, 24, 1.5, (40.0, 16, (16.0, 8, 2.0, 0.5)), 5, 1, ff=16)],
    "torch_dtype": "bfloat16",
}

ALL = {"bat_a": BAT_A, "bat_b": BAT_B, "bat_c": BAT_C}
