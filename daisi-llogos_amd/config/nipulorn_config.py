"""Typed configuration of the Nipulorn decoder, read from its config.json.

The file names the design in `architecture`, gives the model-wide sizes and constants (`vocab`,
`width`, `embedding.scale`, `logit_scale`, `norm.eps`, `canon.taps`) and lists the layers: each
entry has a `type` (which mixer), the mixer's sizes under `mixer` and the feed-forward under `mlp`
(null: the layer has none).  One size is not in the file, the rank of the recurrent mixer's decay
projection: it is the first dimension of the layer's `mix.w1` tensor, so the reader takes the
checkpoint's tensor shapes too when there is a checkpoint (a `decay_rank` key in the mixer's entry
serves where there is none: random weights)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from .model_config import ConfigError, ConfigReader


@dataclass(frozen=True)
class YarnScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class WkvMixerConfig:
    heads: int
    dim: int
    decay_rank: int


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int            # unrotated query/key dimensions a head
    rot_dim: int        # rotated ones
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_dims: int       # how many of the rot_dim dimensions are rotated
    rot_base: float
    rot_scaling: Optional[YarnScaling]


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class NipulornLayerConfig:
    type: str
    mixer: object
    mlp: Optional[DenseMlpConfig]


@dataclass(frozen=True)
class NipulornConfig:
    architecture: str
    vocab: int
    width: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    canon_taps: int
    layers: Tuple[NipulornLayerConfig, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    @classmethod
    def from_dict(cls, data: dict, shapes: Optional[Dict[str, tuple]] = None) -> "NipulornConfig":
        r = ConfigReader(data)
        width = r.int("width")
        layers = []
        raw = r._raw("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a list with at least one layer")
        for i, entry in enumerate(raw):
            where = f"config.json layers[{i}]"
            lr = ConfigReader(entry, where)
            kind = lr.str("type")
            mr = ConfigReader(lr.obj("mixer"), where + ".mixer")
            if kind == "wkv":
                rank = mr.int("decay_rank", None)
                name = f"l{i}.mix.w1"
                if rank is None and shapes is not None and name in shapes:
                    rank = int(shapes[name][0])
                if rank is None:
                    rank = max(16, width // 16)
                mixer = WkvMixerConfig(mr.int("heads"), mr.int("dim"), rank)
            elif kind == "latent_attention":
                rot = ConfigReader(mr.obj("rot"), where + ".mixer.rot")
                sc = rot.obj("scaling", None)
                scaling = None
                if sc is not None:
                    sr = ConfigReader(sc, where + ".mixer.rot.scaling")
                    scaling = YarnScaling(sr.float("factor"), sr.float("original"), sr.float("fast"), sr.float("slow"))
                mixer = LatentAttentionConfig(mr.int("heads"), mr.int("dim"), mr.int("rot_dim"), mr.int("vdim"), mr.int("q_rank"),
                                              mr.int("kv_rank"), mr.float("scale"), rot.int("dims"), rot.float("base"), scaling)
                if mixer.rot_dims % 2 or not 0 <= mixer.rot_dims <= mixer.rot_dim:
                    raise ConfigError(f"{where}: rot.dims {mixer.rot_dims} must be even and within rot_dim {mixer.rot_dim}")
            else:
                raise ConfigError(f"{where}: unknown layer type '{kind}' (wkv, latent_attention)")
            if min(mixer.heads, mixer.dim) <= 0:
                raise ConfigError(f"{where}: heads and dim must be positive")
            mlp = lr.obj("mlp", None)
            if mlp is not None:
                fr = ConfigReader(mlp, where + ".mlp")
                if fr.str("kind") != "dense":
                    raise ConfigError(f"{where}: unknown feed-forward kind '{fr.str('kind')}' (dense)")
                mlp = DenseMlpConfig(fr.int("ff"))
            layers.append(NipulornLayerConfig(kind, mixer, mlp))
        emb = ConfigReader(r.obj("embedding"), "config.json embedding")
        norm = ConfigReader(r.obj("norm"), "config.json norm")
        canon = ConfigReader(r.obj("canon"), "config.json canon")
        cfg = cls(r.str("architecture", "Nipulorn"), r.int("vocab"), width, emb.float("scale"), r.float("logit_scale"),
                  norm.float("eps"), canon.int("taps"), tuple(layers))
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.canon_taps < 1:
            raise ConfigError("config.json: vocab, width and canon.taps must be positive")
        return cfg
