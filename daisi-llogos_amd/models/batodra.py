"""The Batodra decoder as a ModelSpec: blocks whose norm comes after the residual sum
(`x <- norm(alpha x + sublayer(x))`, the sublayers read the stream itself), whose mixer is a gated linear
recurrence, differential attention, or attention over a window that keeps the first tokens, and whose
feed-forward is two matrices around the square of relu.  A layer may use an earlier layer's tensors: it is
then a second run of that layer in the schedule, with cache units of its own.

Tensor names: `embed`, `head`, `final.norm`, and per layer i that owns tensors `l<i>.norm1`, `l<i>.norm2`,
`l<i>.mix.*`, `l<i>.mlp.{up,down}` (no `.weight` suffix)."""
from __future__ import annotations

from ..config.batodra_config import BatodraConfig
from .model import LayerSpec, ModelSpec, ScheduleEntry

DECAY_SHARPNESS = 8.0        # the recurrence's decay is exp(-8 r softplus(lam))


def _rotary(rot, dim: int):
    """The rotation of a mixer's queries and keys as a position encoding, or None when nothing is rotated."""
    from ..parts.base import POSITIONS, make
    if rot is None:
        return None
    scaling = None
    if rot.scaling is not None:
        factor, original, fast, slow = rot.scaling
        scaling = {"type": "yarn", "factor": factor, "original": original, "fast": fast, "slow": slow}
    return make(POSITIONS, "position encoding", "rotary", head_dim=dim, rot=rot.dims, theta=rot.base, pairing="split_half",
                scaling=scaling)


def batodra_spec(cfg: BatodraConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps

    def norm(name: str):
        return ("rmsnorm", dict(name=name, width=W, eps=eps, suffix=""))

    layers, index_of, schedule = [], {}, []
    for i, L in enumerate(cfg.layers):
        if L.weights_of is not None:
            schedule.append(ScheduleEntry(index_of[L.weights_of]))
            continue
        p, m = f"l{i}.", L.mixer
        if L.type == "rglru":
            mixer = ("rglru", dict(prefix=p + "mix.", hidden=W, width=m.width, blocks=m.blocks, conv_taps=m.conv,
                                   sharpness=DECAY_SHARPNESS))
        else:
            position = _rotary(m.rot, m.dim)
            if L.type == "attention":
                mixer = ("diff_attention", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                                                v_dim=m.vdim, scale=m.scale, diff=m.diff, position=position, eps=eps,
                                                window=m.window, sinks=m.keep_first))
            else:
                mixer = ("attention", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                                           v_dim=m.vdim, scale=m.scale, position=position, eps=eps, window=m.window,
                                           sinks=m.keep_first, unit_qk=True, names=("q", "k", "v", "o"), suffix=""))
        spec = LayerSpec(mixer=mixer, mixer_norm=norm(p + "norm1"), block="post_norm", options=dict(alpha=cfg.alpha))
        if L.second_norm:
            spec.ffn_norm = norm(p + "norm2")
        if L.ff:
            spec.ffn = ("activated", dict(prefix=p + "mlp.", hidden=W, intermediate=L.ff, activation="relu2", suffix=""))
        index_of[i] = len(layers)
        layers.append(spec)
        schedule.append(ScheduleEntry(index_of[i]))
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=W, embed_name="embed", layers=layers, final_norm=norm("final.norm"),
                     head_name="head", head_suffix="", schedule=schedule)
