"""The Zogurax decoder as a ModelSpec: parallel blocks (one layer norm; the mixer and the
feed-forward both read it and both add to the stream), whose mixer is softmax attention without a
rotation in one of two forms and whose feed-forward is a mixture of experts chosen by a table over
token ids with a gated shared expert.  A position vector of sines and cosines is added to the
embedding.  A run of layers may be gone through several times with the same weights and a cache of
its own each time; at the head of every pass the stream and the embedding output go through a
matrix together and the pass's own vector is added.

Tensor names: `embed`, `head`, `final.norm`, `loop.in`, `loop.step`, and per layer i `l<i>.norm1`,
`l<i>.mix.{q,k,v,o}` (+ `.b` biases, `.conv` taps, `.norm` weights), `l<i>.mix.g`,
`l<i>.mlp.e<j>.{up,down}`, `l<i>.mlp.table`, `l<i>.mlp.shared.{up,down,sg}` (no `.weight` suffix)."""
from __future__ import annotations

from ..config.zogurax_config import ZoguraxConfig
from .model import LayerSpec, ModelSpec, ScheduleEntry

POSITION_BASE = 10000.0


def zogurax_spec(cfg: ZoguraxConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps

    def norm(name: str):
        return ("layernorm", dict(name=name, width=W, eps=eps, suffix=""))

    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        second = L.type == "attention_2"
        mixer = ("capped_attention", dict(
            prefix=p + "mix.", hidden=W, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, v_dim=m.vdim, scale=m.scale,
            softcap=m.softcap, temp_coef=m.temp_coef, temp_every=m.temp_every, eps=eps,
            bias=second, unit_sink=second, conv_taps=0 if second else m.conv, whole_norm=not second, head_gate=not second))
        spec = LayerSpec(mixer=mixer, mixer_norm=norm(p + "norm1"), block="parallel")
        if L.mlp is not None:
            f = L.mlp
            spec.ffn = ("table_moe", dict(prefix=p + "mlp.", hidden=W, vocab=cfg.vocab, n_experts=f.experts, top=f.top,
                                          intermediate=f.ff, shared_intermediate=f.shared_ff, activation="relu2"))
        layers.append(spec)
    schedule, parts = None, []
    if cfg.loop is not None:
        lp = cfg.loop
        parts.append(("part", "loop_entry", dict(matrix="loop.in", steps="loop.step", width=W, times=lp.times)))
        schedule = [ScheduleEntry(i) for i in range(lp.start)]
        for t in range(lp.times):
            schedule += [ScheduleEntry(i, enter=(0, t) if i == lp.start else None) for i in range(lp.start, lp.stop)]
        schedule += [ScheduleEntry(i) for i in range(lp.stop, len(layers))]
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=W, embed_name="embed", layers=layers, final_norm=norm("final.norm"),
                     head_name="head", head_suffix="", schedule=schedule, stream_parts=parts, position_vector=POSITION_BASE)
