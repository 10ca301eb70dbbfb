"""The Zasidra decoder as a ModelSpec: blocks whose norm stands on each sublayer's output alone
(`x <- x + norm(sublayer(x))`, the sublayers read the stream itself), whose mixer is grouped-query attention
with norms over the whole of q and of k, a partial rotation and a learned sink, or attention through a
latent with a gate on every head, and whose feed-forward is SwiGLU or a mixture of SwiGLU experts chosen by
a router.  An attention layer may read an earlier layer's keys and values: its run in the schedule names
that layer's run as the owner of its cache.

Tensor names: `embed`, `head`, `final.norm`, and per layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,correction,e<j>.{gate,up,down},shared.{gate,up,down}}`
(no `.weight` suffix).  The norms' weights are stored as their distance from one."""
from __future__ import annotations

from ..config.zasidra_config import ZasidraConfig
from .model import LayerSpec, ModelSpec, ScheduleEntry


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


def zasidra_spec(cfg: ZasidraConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps

    def norm(name: str):
        return ("rmsnorm", dict(name=name, width=W, eps=eps, offset=1.0, suffix=""))

    layers, schedule = [], []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        if L.type == "attention":
            mixer = ("capped_attention", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                                              v_dim=m.vdim, scale=m.scale, eps=eps, whole_norm=True, learned_sink=True,
                                              position=_rotary(m.rot, m.dim), own_kv=m.kv_from is None))
            schedule.append(ScheduleEntry(i, cache_of=m.kv_from))
        else:
            mixer = ("latent_attention", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, dim=m.dim, rot_dim=0, v_dim=m.vdim,
                                              q_rank=0, kv_rank=m.kv_rank, scale=m.scale, eps=eps, sink=False, head_gate=True))
            schedule.append(ScheduleEntry(i))
        spec = LayerSpec(mixer=mixer, mixer_norm=norm(p + "norm1"), block="output_norm")
        if L.mlp is not None:
            spec.ffn_norm = norm(p + "norm2")
            if L.mlp.kind == "dense":
                spec.ffn = ("swiglu", dict(prefix=p + "mlp.", hidden=W, intermediate=L.mlp.ff, names=("gate", "up", "down"), suffix=""))
            else:
                r = L.mlp.router
                spec.ffn = ("routed_moe", dict(prefix=p + "mlp.", hidden=W, n_experts=r.experts, identity=r.identity, top=r.top,
                                               intermediate=L.mlp.ff, groups=r.groups, keep=r.keep, scale=r.scale,
                                               shared_intermediate=L.mlp.shared_ff))
        layers.append(spec)
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=W, embed_name="embed", layers=layers, final_norm=norm("final.norm"),
                     head_name="head", head_suffix="", schedule=schedule, embed_scale=cfg.embedding_scale)
