"""Small configurations of the Zasidra design for tests.  Between them every size differs from layer
to layer and from the others of its layer (heads, key/value heads equal to the heads, half of them and
one; key and value widths that differ either way; widths and ranks that are no multiple of 16), the two
layer types come in several orders, a layer reads the keys and values of the layer right before it, of
one several layers back, or two layers read the same one; rotations cover a part of a head or all of
it, with and without stretched frequencies; the feed-forward is absent, dense or a mixture whose router
has groups or none, keeps all groups or some, has outputs without matrices or none, one choice or all
of the outputs, a shared expert or none."""


def rot(dims, base, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def attention(heads, kv_heads, dim, vdim, scale, rotation=None, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rotation is not None:
        m["rot"] = rotation
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, vdim, kv_rank, scale, mlp=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, scale, groups=None, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if identity:
        r["identity"] = identity
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        m["shared"] = {"ff": shared}
    return m


YARN = (8.0, 64, 16.0, 2.0)       # stretched frequencies whose ramp lies within a test's length

ZAS_A = {   # attention first; its keys and values are read two layers on; 4 groups of which 2 are kept; outputs without matrices
    "architecture": "Zasidra", "vocab": 199, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.5},
    "layers": [attention(4, 2, 32, 48, 0.3, rot(16, 10000.0, YARN), mlp=moe(6, 2, 3, 40, 1.7, groups=(4, 2), shared=24)),
               latent(3, 24, 40, 48, 0.25, mlp=dense(136)),
               attention(4, 2, 32, 48, 0.2, rot(16, 10000.0, YARN), kv_from=0, mlp=None),
               latent(5, 16, 8, 20, 0.4, mlp=moe(5, 0, 2, 24, 0.8, groups=None, shared=56))],
    "torch_dtype": "bfloat16",
}

ZAS_B = {   # latent first; widths that are no multiple of 16; a whole head rotated, plain frequencies; kv heads = heads; one group
    "architecture": "Zasidra", "vocab": 130, "width": 72, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
    "layers": [latent(2, 40, 24, 24, 0.3, mlp=moe(3, 1, 4, 20, 1.0, groups=(1, 1))),
               attention(3, 3, 24, 40, 0.35, rot(24, 500.0), mlp=dense(50)),
               attention(3, 3, 24, 40, 0.3, rot(24, 500.0), kv_from=1, mlp=moe(2, 0, 1, 30, 2.0, groups=(2, 1))),
               attention(5, 1, 8, 16, 0.5, None, mlp=None)],
    "torch_dtype": "bfloat16",
}

ZAS_C = {   # head shapes that the matrix-core kernels take; two layers read the same keys and values; 16 query heads a kv head
    "architecture": "Zasidra", "vocab": 190, "width": 128, "norm": {"eps": 1e-5}, "embedding": {"scale": 4.0},
    "layers": [latent(4, 64, 64, 64, 0.12, mlp=dense(96)),
               attention(4, 2, 64, 128, 0.12, rot(32, 20000.0, (4.0, 128, 8.0, 1.0)), mlp=moe(8, 4, 3, 64, 1.2, groups=(3, 2), shared=32)),
               attention(16, 1, 128, 64, 0.09, rot(64, 1000000.0), mlp=moe(4, 0, 4, 32, 1.0)),
               attention(4, 2, 64, 128, 0.1, rot(32, 20000.0, (4.0, 128, 8.0, 1.0)), kv_from=1, mlp=dense(64)),
               latent(2, 128, 96, 128, 0.09, mlp=None),
               attention(4, 2, 64, 128, 0.15, rot(32, 20000.0, (4.0, 128, 8.0, 1.0)), kv_from=1, mlp=moe(2, 2, 2, 48, 0.5, groups=(2, 2)))],
    "torch_dtype": "bfloat16",
}

ZAS_D = {   # a reader right behind its owner; one head; an expert alone beside an output without matrices; no embedding scale given
    "architecture": "Zasidra", "vocab": 67, "width": 48, "norm": {"eps": 1e-5},
    "layers": [attention(1, 1, 16, 16, 0.4, rot(2, 100.0, (2.0, 16, 4.0, 1.0)), mlp=moe(1, 1, 1, 24, 3.0)),
               attention(1, 1, 16, 16, 0.5, rot(2, 100.0, (2.0, 16, 4.0, 1.0)), kv_from=0, mlp=dense(24))],
    "torch_dtype": "bfloat16",
}

ALL = {"zas_a": ZAS_A, "zas_b": ZAS_B, "zas_c": ZAS_C, "zas_d": ZAS_D}
