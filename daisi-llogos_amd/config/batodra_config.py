"""Typed configuration of the Batodra decoder, read from its config.json.

The file names the design in `architecture`, gives `vocab`, `width`, `norm.eps` and `postln_alpha`
(the factor on the stream in every residual sum; the norm comes after the sum), and lists the layers.
A layer entry has a `type`, the mixer's sizes and constants under `mixer`, its feed-forward under
`mlp` (null: none; `kind` 'dense' with `ff`) and optionally `weights_of`: the number of an earlier
layer whose tensors it uses, with a cache or state of its own.

    'rglru'        width, blocks, conv (taps)
    'attention'    heads, kv_heads, dim, vdim, scale, diff, rot.base, rot.dims            (differential attention)
    'attention_2'  heads, kv_heads, dim, vdim, scale, rot.base, rot.dims, rot.scaling.{factor, original, fast, slow},
                   mask.size, mask.keep_first                                             (window that keeps the first tokens)

Whether a layer without a feed-forward still has its second norm is left to the checkpoint: the reader
takes the tensors' shapes and looks for `l<i>.norm2`."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from .model_config import ConfigError, ConfigReader

LAYER_TYPES = ("rglru", "attention", "attention_2")


@dataclass(frozen=True)
class BatodraRecurrent:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class BatodraRotation:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]]     # (factor, original, fast, slow) of the YaRN rule, or None


@dataclass(frozen=True)
class BatodraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[BatodraRotation]
    diff: float = 0.0          # 'attention' only
    window: int = 0            # 0: every earlier token is seen
    keep_first: int = 0


@dataclass(frozen=True)
class BatodraLayer:
    type: str
    mixer: object              # BatodraRecurrent or BatodraAttention
    ff: int                    # 0: no feed-forward
    weights_of: Optional[int]  # the layer whose tensors this one uses
    second_norm: bool          # the norm behind the feed-forward's sum (always with a feed-forward)

    @property
    def owner(self) -> Optional[int]:
        return self.weights_of


@dataclass(frozen=True)
class BatodraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    alpha: float
    layers: Tuple[BatodraLayer, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    @classmethod
    def from_dict(cls, data: dict, shapes: Optional[Dict[str, tuple]] = None) -> "BatodraConfig":
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
            mixer = _recurrent(mr, where) if kind == "rglru" else _attention(mr, where, kind)
            ff = 0
            mlp = lr.obj("mlp", None)
            if mlp is not None:
                fr = ConfigReader(mlp, where + ".mlp")
                if fr.str("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp: unknown feed-forward kind '{fr.str('kind')}' (dense)")
                ff = fr.int("ff")
                if ff <= 0:
                    raise ConfigError(f"{where}.mlp: ff must be positive")
            src = lr.int("weights_of", None)
            if src is not None:
                if not 0 <= src < i:
                    raise ConfigError(f"{where}: weights_of must name an earlier layer, got {src}")
                if layers[src].weights_of is not None:
                    src = layers[src].weights_of               # a borrower of a borrower uses the owner's
                own = layers[src]
                if own.type != kind or own.mixer != mixer or own.ff != ff:
                    raise ConfigError(f"{where}: a layer that uses layer {src}'s tensors must have its type and sizes")
            owner = i if src is None else src
            second = ff > 0 or (shapes is not None and f"l{owner}.norm2" in shapes)
            layers.append(BatodraLayer(kind, mixer, ff, src, second))
        norm = ConfigReader(r.obj("norm"), "config.json norm")
        cfg = cls(r.str("architecture", "Batodra"), r.int("vocab"), r.int("width"), norm.float("eps"),
                  r.float("postln_alpha", 1.0), tuple(layers))
        if cfg.vocab <= 0 or cfg.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg


def _recurrent(mr: ConfigReader, where: str) -> BatodraRecurrent:
    m = BatodraRecurrent(mr.int("width"), mr.int("blocks", 1), mr.int("conv", 1))
    if m.width <= 0 or m.blocks <= 0 or m.width % m.blocks or m.conv < 1:
        raise ConfigError(f"{where}.mixer: width must be a positive multiple of blocks, conv at least 1")
    return m


def _attention(mr: ConfigReader, where: str, kind: str) -> BatodraAttention:
    heads = mr.int("heads")
    dim = mr.int("dim")
    rot = None
    ro = mr.obj("rot", None)
    if ro is not None:
        rr = ConfigReader(ro, where + ".mixer.rot")
        scaling = None
        so = rr.obj("scaling", None)
        if so is not None:
            sr = ConfigReader(so, where + ".mixer.rot.scaling")
            scaling = (sr.float("factor"), sr.float("original"), sr.float("fast"), sr.float("slow"))
        rot = BatodraRotation(rr.float("base"), rr.int("dims"), scaling)
        if rot.dims < 0 or rot.dims % 2 or rot.dims > dim or rot.base <= 0:
            raise ConfigError(f"{where}.mixer.rot: dims must be even and within dim, base positive")
        if rot.dims == 0:
            rot = None
    window = keep = 0
    mo = mr.obj("mask", None)
    if mo is not None:
        kr = ConfigReader(mo, where + ".mixer.mask")
        window, keep = kr.int("size", 0), kr.int("keep_first", 0)
        if window < 0 or keep < 0:
            raise ConfigError(f"{where}.mixer.mask: size and keep_first must not be negative")
    m = BatodraAttention(heads, mr.int("kv_heads", heads), dim, mr.int("vdim", dim), mr.float("scale"), rot,
                         mr.float("diff") if kind == "attention" else 0.0, window, keep)
    if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
        raise ConfigError(f"{where}.mixer: heads, kv_heads, dim and vdim must be positive, heads a multiple of kv_heads")
    return m
