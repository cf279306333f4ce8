"""The Nipulorn decoder as a ModelSpec: sandwich blocks (a norm before and after each sublayer, a
short convolution over time on what a sublayer reads), whose mixer is a recurrence with a matrix
state ('wkv') or attention through a latent ('latent_attention'), layer by layer as the
configuration lists them; some layers have a feed-forward with the xIELU activation.  The norms'
weights are stored as offsets from one; the embedding is scaled on the way in and serves, unscaled,
as the output head, whose logits are scaled.

Tensor names: `embed`, `final.norm`, and per layer i `l<i>.norm1`, `.norm1b`, `.norm2`, `.norm2b`,
`.canon1`, `.canon2`, `.mix.*`, `.mlp.up`, `.mlp.down`, `.mlp.act` (no `.weight` suffix)."""
from __future__ import annotations

from ..config.nipulorn_config import NipulornConfig
from ..parts.rope import Rotary
from .model import LayerSpec, ModelSpec


def nipulorn_spec(cfg: NipulornConfig) -> ModelSpec:
    W, eps = cfg.width, cfg.norm_eps

    def norm(name: str):
        return ("rmsnorm", dict(name=name, width=W, eps=eps, offset=1.0, suffix=""))

    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L.mixer
        if L.type == "wkv":
            mixer = ("wkv", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, head_dim=m.dim, decay_rank=m.decay_rank, eps=eps))
        else:
            position = None
            if m.rot_dims:
                scaling = None
                if m.rot_scaling is not None:
                    s = m.rot_scaling
                    scaling = dict(type="yarn", factor=s.factor, original=s.original, fast=s.fast, slow=s.slow)
                position = Rotary(m.rot_dim, m.rot_dims, m.rot_base, pairing="interleaved", scaling=scaling)
            mixer = ("latent_attention", dict(prefix=p + "mix.", hidden=W, n_heads=m.heads, dim=m.dim, rot_dim=m.rot_dim,
                                              v_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=eps,
                                              position=position))
        more = {"post_mixer_norm": ("norm",) + norm(p + "norm1b")}
        if cfg.canon_taps >= 1:
            more["mixer_conv"] = ("part", "causal_conv", dict(name=p + "canon1", width=W, taps=cfg.canon_taps))
        spec = LayerSpec(mixer=mixer, mixer_norm=norm(p + "norm1"), block="sandwich", more=more)
        if L.mlp is not None:
            spec.ffn = ("activated", dict(prefix=p + "mlp.", hidden=W, intermediate=L.mlp.ff, activation="xielu"))
            spec.ffn_norm = norm(p + "norm2")
            more["post_ffn_norm"] = ("norm",) + norm(p + "norm2b")
            if cfg.canon_taps >= 1:
                more["ffn_conv"] = ("part", "causal_conv", dict(name=p + "canon2", width=W, taps=cfg.canon_taps))
        layers.append(spec)
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=W, embed_name="embed", layers=layers,
                     final_norm=norm("final.norm"), head_name="embed", tie_head=True,
                     embed_scale=cfg.embedding_scale, logit_scale=cfg.logit_scale)
