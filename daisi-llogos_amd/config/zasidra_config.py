"""Typed configuration of the Zasidra decoder, read from its config.json.

The file names the design in `architecture`, gives `vocab`, `width`, `norm.eps` and `embedding.scale`,
and lists the layers.  A layer entry has a `type`, the mixer's sizes and constants under `mixer`, and
its feed-forward under `mlp` (null: none).

    'attention'         heads, kv_heads, dim, vdim, scale, rot.{base, dims, scaling.{factor, original, fast, slow}},
                        kv_from (an earlier attention layer whose keys and values this layer reads; it then
                        has no key or value tensors of its own)
    'latent_attention'  heads, dim, vdim, kv_rank, scale

    mlp.kind 'dense'    ff
    mlp.kind 'moe'      expert.ff, shared.ff (optional), router.{experts, top, scale, identity,
                        groups.{count, keep}}: the router has experts + identity outputs, the last
                        `identity` of which return their input
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .model_config import ConfigError, ConfigReader

LAYER_TYPES = ("attention", "latent_attention")


@dataclass(frozen=True)
class ZasidraRotation:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]]     # (factor, original, fast, slow) of the YaRN rule, or None


@dataclass(frozen=True)
class ZasidraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[ZasidraRotation]
    kv_from: Optional[int]       # the layer whose keys and values this one reads


@dataclass(frozen=True)
class ZasidraLatent:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float


@dataclass(frozen=True)
class ZasidraRouter:
    experts: int                 # experts with matrices
    identity: int                # router outputs behind them that return their input
    top: int
    scale: float
    groups: int                  # 1: no groups
    keep: int

    @property
    def outputs(self) -> int:
        return self.experts + self.identity


@dataclass(frozen=True)
class ZasidraMlp:
    kind: str                    # 'dense' or 'moe'
    ff: int                      # dense: the width between the matrices; moe: an expert's
    router: Optional[ZasidraRouter] = None
    shared_ff: int = 0           # moe: the shared expert's width (0: none)


@dataclass(frozen=True)
class ZasidraLayer:
    type: str
    mixer: object                # ZasidraAttention or ZasidraLatent
    mlp: Optional[ZasidraMlp]


@dataclass(frozen=True)
class ZasidraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: Tuple[ZasidraLayer, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    @classmethod
    def from_dict(cls, data: dict) -> "ZasidraConfig":
        r = ConfigReader(data)
        raw = r._raw("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(raw):
            where = f"config.json layers[{i}]"
            lr = ConfigReader(entry, where)
            kind = lr.str("type")
            if kind not in LAYER_TYPES:
                raise ConfigError(f"{where}: unknown layer type '{kind}' ({', '.join(LAYER_TYPES)})")
            mr = ConfigReader(lr.obj("mixer"), where + ".mixer")
            mixer = _attention(mr, where, layers) if kind == "attention" else _latent(mr, where)
            mlp = lr.obj("mlp", None)
            layers.append(ZasidraLayer(kind, mixer, _mlp(ConfigReader(mlp, where + ".mlp"), where) if mlp is not None else None))
        norm = ConfigReader(r.obj("norm"), "config.json norm")
        emb = r.obj("embedding", None)
        scale = ConfigReader(emb, "config.json embedding").float("scale", 1.0) if emb is not None else 1.0
        cfg = cls(r.str("architecture", "Zasidra"), r.int("vocab"), r.int("width"), norm.float("eps"), scale, tuple(layers))
        if cfg.vocab <= 0 or cfg.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg


def _rotation(mr: ConfigReader, where: str, dim: int) -> Optional[ZasidraRotation]:
    ro = mr.obj("rot", None)
    if ro is None:
        return None
    rr = ConfigReader(ro, where + ".mixer.rot")
    scaling = None
    so = rr.obj("scaling", None)
    if so is not None:
        sr = ConfigReader(so, where + ".mixer.rot.scaling")
        scaling = (sr.float("factor"), sr.float("original"), sr.float("fast"), sr.float("slow"))
        if scaling[0] <= 0 or scaling[1] <= 0 or scaling[2] <= 0 or scaling[3] <= 0:
            raise ConfigError(f"{where}.mixer.rot.scaling: factor, original, fast and slow must be positive")
    rot = ZasidraRotation(rr.float("base"), rr.int("dims"), scaling)
    if rot.dims < 0 or rot.dims % 2 or rot.dims > dim or rot.base <= 0:
        raise ConfigError(f"{where}.mixer.rot: dims must be even and within dim, base positive")
    return rot if rot.dims else None


def _attention(mr: ConfigReader, where: str, before: list) -> ZasidraAttention:
    heads, dim = mr.int("heads"), mr.int("dim")
    m = ZasidraAttention(heads, mr.int("kv_heads", heads), dim, mr.int("vdim", dim), mr.float("scale"),
                         _rotation(mr, where, dim), mr.int("kv_from", None))
    if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
        raise ConfigError(f"{where}.mixer: heads, kv_heads, dim and vdim must be positive, heads a multiple of kv_heads")
    if m.kv_from is not None:
        if not 0 <= m.kv_from < len(before) or before[m.kv_from].type != "attention":
            raise ConfigError(f"{where}.mixer: kv_from must name an earlier attention layer, got {m.kv_from}")
        own = before[m.kv_from].mixer
        if own.kv_from is not None:
            raise ConfigError(f"{where}.mixer: kv_from names layer {m.kv_from}, which has no keys and values of its own")
        if (own.kv_heads, own.dim, own.vdim, own.rot) != (m.kv_heads, m.dim, m.vdim, m.rot):
            raise ConfigError(f"{where}.mixer: kv_from names layer {m.kv_from}, whose kv_heads, dim, vdim or rot differ from this layer's")
    return m


def _latent(mr: ConfigReader, where: str) -> ZasidraLatent:
    dim = mr.int("dim")
    m = ZasidraLatent(mr.int("heads"), dim, mr.int("vdim", dim), mr.int("kv_rank"), mr.float("scale"))
    if min(m.heads, m.dim, m.vdim, m.kv_rank) <= 0:
        raise ConfigError(f"{where}.mixer: heads, dim, vdim and kv_rank must be positive")
    return m


def _mlp(fr: ConfigReader, where: str) -> ZasidraMlp:
    kind = fr.str("kind", "dense")
    if kind == "dense":
        ff = fr.int("ff")
        if ff <= 0:
            raise ConfigError(f"{where}.mlp: ff must be positive")
        return ZasidraMlp("dense", ff)
    if kind != "moe":
        raise ConfigError(f"{where}.mlp: unknown feed-forward kind '{kind}' (dense, moe)")
    ff = ConfigReader(fr.obj("expert"), where + ".mlp.expert").int("ff")
    rr = ConfigReader(fr.obj("router"), where + ".mlp.router")
    groups, keep = 1, 1
    go = rr.obj("groups", None)
    if go is not None:
        gr = ConfigReader(go, where + ".mlp.router.groups")
        groups = gr.int("count", 1)
        keep = gr.int("keep", groups)
    router = ZasidraRouter(rr.int("experts"), rr.int("identity", 0), rr.int("top"), rr.float("scale", 1.0), groups, keep)
    if ff <= 0 or router.experts < 0 or router.identity < 0 or router.outputs <= 0 or not 1 <= router.top <= router.outputs:
        raise ConfigError(f"{where}.mlp: expert.ff and the router's outputs must be positive, top within them")
    if groups < 1 or router.outputs % groups or not 1 <= keep <= groups:
        raise ConfigError(f"{where}.mlp.router.groups: count must divide experts + identity, keep lie within 1..count")
    if keep * (router.outputs // groups) < router.top:
        raise ConfigError(f"{where}.mlp.router: the {keep} kept groups hold fewer than top = {router.top} outputs")
    shared = 0
    so = fr.obj("shared", None)
    if so is not None:
        shared = ConfigReader(so, where + ".mlp.shared").int("ff")
        if shared <= 0:
            raise ConfigError(f"{where}.mlp.shared: ff must be positive")
    return ZasidraMlp("moe", ff, router, shared)
