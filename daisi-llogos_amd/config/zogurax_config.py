"""Typed configuration of the Zogurax decoder, read from its config.json.

The file names the design in `architecture`, gives `vocab`, `width` and `norm.eps`, lists the
layers and, under `loop`, which run of layers is gone through several times.  A layer entry has a
`type` ('attention': projections without biases, a short convolution over time behind them, a
norm over the whole of q and of k, a gate on every head's output; 'attention_2': projections
with biases and a softmax with one added to its denominator), the mixer's sizes and constants
under `mixer` (`heads`, `kv_heads`, `dim`, `vdim`, `scale`, `softcap`, `q_temp.coef` /
`q_temp.every`, `conv` taps) and its feed-forward under `mlp` (null: none): `kind` 'moe' with
`router.experts` / `router.top`, `expert.ff` and `shared.ff`."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .model_config import ConfigError, ConfigReader

LAYER_TYPES = ("attention", "attention_2")


@dataclass(frozen=True)
class ZoguraxMixerConfig:
    heads: int
    kv_heads: int
    dim: int            # query/key dimensions a head
    vdim: int           # value dimensions a head
    scale: float
    softcap: float      # 0: scores are not bent
    temp_coef: float    # 0: no factor on the query
    temp_every: int
    conv: int           # taps of the convolution behind the projections ('attention' only; 0: none)


@dataclass(frozen=True)
class ZoguraxMlpConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int      # 0: no shared expert


@dataclass(frozen=True)
class ZoguraxLayerConfig:
    type: str
    mixer: ZoguraxMixerConfig
    mlp: Optional[ZoguraxMlpConfig]


@dataclass(frozen=True)
class ZoguraxLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class ZoguraxConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[ZoguraxLayerConfig, ...]
    loop: Optional[ZoguraxLoop]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    @classmethod
    def from_dict(cls, data: dict) -> "ZoguraxConfig":
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
            coef, every = 0.0, 1
            temp = mr.obj("q_temp", None)
            if temp is not None:
                tr = ConfigReader(temp, where + ".mixer.q_temp")
                coef, every = tr.float("coef"), tr.int("every")
                if every < 1:
                    raise ConfigError(f"{where}.mixer.q_temp: every must be at least 1")
            heads = mr.int("heads")
            mixer = ZoguraxMixerConfig(heads, mr.int("kv_heads", heads), mr.int("dim"), mr.int("vdim"), mr.float("scale"),
                                       mr.float("softcap", 0.0), coef, every,
                                       mr.int("conv", 0) if kind == "attention" else 0)
            if min(mixer.heads, mixer.kv_heads, mixer.dim, mixer.vdim) <= 0 or mixer.heads % mixer.kv_heads:
                raise ConfigError(f"{where}.mixer: heads, kv_heads, dim and vdim must be positive, heads a multiple of kv_heads")
            if mixer.softcap < 0 or mixer.conv < 0:
                raise ConfigError(f"{where}.mixer: softcap and conv must not be negative")
            mlp = lr.obj("mlp", None)
            if mlp is not None:
                fr = ConfigReader(mlp, where + ".mlp")
                if fr.str("kind") != "moe":
                    raise ConfigError(f"{where}.mlp: unknown feed-forward kind '{fr.str('kind')}' (moe)")
                rr = ConfigReader(fr.obj("router"), where + ".mlp.router")
                er = ConfigReader(fr.obj("expert"), where + ".mlp.expert")
                shared = fr.obj("shared", None)
                shared_ff = ConfigReader(shared, where + ".mlp.shared").int("ff") if shared is not None else 0
                mlp = ZoguraxMlpConfig(rr.int("experts"), rr.int("top"), er.int("ff"), shared_ff)
                if not 1 <= mlp.top <= mlp.experts or mlp.ff <= 0 or mlp.shared_ff < 0:
                    raise ConfigError(f"{where}.mlp: top must lie in 1..experts, ff must be positive")
            layers.append(ZoguraxLayerConfig(kind, mixer, mlp))
        loop = r.obj("loop", None)
        if loop is not None:
            pr = ConfigReader(loop, "config.json loop")
            loop = ZoguraxLoop(pr.int("start"), pr.int("stop"), pr.int("times"))
            if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 1:
                raise ConfigError(f"config.json loop: start <= stop within the {len(layers)} layers and times >= 1, "
                                  f"got {loop.start}, {loop.stop}, {loop.times}")
            if loop.start == loop.stop:
                loop = None
        norm = ConfigReader(r.obj("norm"), "config.json norm")
        cfg = cls(r.str("architecture", "Zogurax"), r.int("vocab"), r.int("width"), norm.float("eps"), tuple(layers), loop)
        if cfg.vocab <= 0 or cfg.width <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg
