"""Typed configuration of the Vupelorn decoder.

config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, optionally
`embedding.bigram` (`buckets`, `mul_prev`, `mul_cur`), and `layers`, one entry a layer: `type` ("gla": gated
linear attention; "latent_attention": attention through a latent with half-split rotary pairs and YaRN scaling;
"latent_attention_2": the same with interleaved pairs, optionally reading another layer's latent, `kv_from`),
`mixer` (the sizes of that type) and `mlp` (`{"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts",
"top"}}` or null).  One size is in no key: the rank of a gated-linear-attention layer's decay projection, which the
shape of its tensor gives (`completed`); `mixer.decay_rank` may state it, which a configuration without a file needs.
Every error names its key.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig, coerce

_REQUIRED = object()


def _get(d, key: str, where: str, kind=int, least=None, default=_REQUIRED):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        if default is not _REQUIRED and isinstance(d, dict):
            return default
        raise ConfigError(f"config.json: required key '{where}.{key}' is missing")
    v = coerce(d[key], f"{where}.{key}", kind)
    if least is not None and v < least:
        raise ConfigError(f"config.json: '{where}.{key}' must be at least {least}, found {v}")
    return v


@dataclass(frozen=True)
class Bigram:
    buckets: int
    mul_prev: int
    mul_cur: int

    @classmethod
    def from_dict(cls, d, where):
        return cls(_get(d, "buckets", where, least=1), _get(d, "mul_prev", where), _get(d, "mul_cur", where))

    def to_dict(self):
        return {"buckets": self.buckets, "mul_cur": self.mul_cur, "mul_prev": self.mul_prev}


@dataclass(frozen=True)
class GlaMixer:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: Optional[int]  # None: the shape of the layer's first decay matrix says it

    @classmethod
    def from_dict(cls, d, where):
        dim = _get(d, "dim", where, least=1)
        c = cls(_get(d, "heads", where, least=1), dim, _get(d, "vdim", where, least=1, default=dim),
                _get(d, "tau", where, float), _get(d, "decay_rank", where, least=1, default=None))
        if not c.tau > 0:
            raise ConfigError(f"config.json: '{where}.tau' must be positive, found {c.tau}")
        return c

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "tau": self.tau, "vdim": self.vdim}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        return d


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float

    def to_dict(self):
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class Rotary:
    base: float
    dims: int
    scaling: Optional[RotaryScaling]

    @classmethod
    def from_dict(cls, d, where, whole: Optional[int] = None):
        """`whole`: the size of the rotated part, which `dims` defaults to."""
        sc = d.get("scaling") if isinstance(d, dict) else None
        scaling = None
        if sc is not None:
            w = where + ".scaling"
            scaling = RotaryScaling(_get(sc, "factor", w, float), _get(sc, "original", w, float),
                                    _get(sc, "fast", w, float), _get(sc, "slow", w, float))
            if not scaling.factor > 0 or not scaling.original > 0 or not scaling.fast > 0 or not scaling.slow > 0:
                raise ConfigError(f"config.json: '{w}' needs positive factor, original, fast and slow")
        c = cls(_get(d, "base", where, float),
                _get(d, "dims", where, least=2, default=_REQUIRED if whole is None else whole), scaling)
        if c.dims % 2 or not c.base > 0:
            raise ConfigError(f"config.json: '{where}.dims' must be even and '{where}.base' positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class LatentMixer:
    heads: int
    dim: int  # unrotated query/key size a head
    rot_dim: int  # rotated query/key size a head (the key's is shared by all heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Rotary
    kv_from: Optional[int]

    @classmethod
    def from_dict(cls, d, where):
        dim = _get(d, "dim", where, least=1)
        rot_dim = _get(d, "rot_dim", where, least=2)
        c = cls(_get(d, "heads", where, least=1), dim, rot_dim,
                _get(d, "vdim", where, least=1, default=dim), _get(d, "kv_rank", where, least=1),
                _get(d, "q_rank", where, least=1), _get(d, "scale", where, float),
                Rotary.from_dict(d.get("rot"), where + ".rot", whole=rot_dim),
                _get(d, "kv_from", where, least=0, default=None))
        if c.rot.dims > c.rot_dim:
            raise ConfigError(f"config.json: '{where}.rot.dims' ({c.rot.dims}) is more than rot_dim ({c.rot_dim})")
        return c

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
             "rot": self.rot.to_dict(), "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class MoE:
    experts: int
    top: int
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d, where):
        if not isinstance(d, dict) or d.get("kind") != "moe":
            raise ConfigError(f"config.json: '{where}.kind' must be 'moe' (or mlp null)")
        c = cls(_get(d.get("router"), "experts", where + ".router", least=1),
                _get(d.get("router"), "top", where + ".router", least=1),
                _get(d.get("expert"), "ff", where + ".expert", least=1),
                _get(d.get("expert"), "limit", where + ".expert", float))
        if c.top > c.experts:
            raise ConfigError(f"config.json: '{where}.router.top' ({c.top}) is more than its {c.experts} experts")
        return c

    def to_dict(self):
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                "router": {"experts": self.experts, "top": self.top}}


LATENT_TYPES = ("latent_attention", "latent_attention_2")


@dataclass(frozen=True)
class VupelornLayer:
    type: str  # "gla" | "latent_attention" | "latent_attention_2"
    gla: Optional[GlaMixer]
    latent: Optional[LatentMixer]
    mlp: Optional[MoE]

    @classmethod
    def from_dict(cls, d, i: int):
        where = f"layers[{i}]"
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        kind, mixer = d.get("type"), d.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"config.json: required key '{where}.mixer' is missing")
        gla = latent = None
        if kind == "gla":
            gla = GlaMixer.from_dict(mixer, where + ".mixer")
        elif kind in LATENT_TYPES:
            latent = LatentMixer.from_dict(mixer, where + ".mixer")
        else:
            raise ConfigError(f"config.json: '{where}.type' must be 'gla', 'latent_attention' or "
                              f"'latent_attention_2', found {kind!r}")
        mlp = d.get("mlp")
        return cls(kind, gla, latent, None if mlp is None else MoE.from_dict(mlp, where + ".mlp"))

    def to_dict(self):
        return {"mixer": (self.gla or self.latent).to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.type}


@dataclass(frozen=True)
class VupelornConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    bigram: Optional[Bigram]
    layers: Tuple[VupelornLayer, ...]
    architecture: str = "Vupelorn"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VupelornConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(VupelornLayer.from_dict(x, i) for i, x in enumerate(layers))
        for i, layer in enumerate(parsed):
            m = layer.latent
            if m is None or m.kv_from is None:
                continue
            j = m.kv_from
            src = parsed[j].latent if 0 <= j < i else None
            if src is None or src.kv_from is not None:
                raise ConfigError(f"config.json: 'layers[{i}].mixer.kv_from' must name an earlier layer that has a "
                                  "latent of its own")
            if (src.kv_rank, src.rot_dim, src.rot) != (m.kv_rank, m.rot_dim, m.rot):
                raise ConfigError(f"config.json: 'layers[{i}]' reads the latent of layer {j} but its kv_rank, rot_dim "
                                  "or rotation differ")
        if not isinstance(d.get("norm"), dict):
            raise ConfigError("config.json: 'norm' must be an object")
        emb = d.get("embedding")
        bigram = emb.get("bigram") if isinstance(emb, dict) else None
        return cls(vocab=_get(d, "vocab", "config", least=1), width=_get(d, "width", "config", least=1),
                   norm_eps=_get(d["norm"], "eps", "norm", float),
                   bigram=None if bigram is None else Bigram.from_dict(bigram, "embedding.bigram"),
                   layers=parsed, architecture=str(d.get("architecture", "Vupelorn")))

    def completed(self, shapes: Mapping[str, Tuple[int, ...]]) -> "VupelornConfig":
        """The sizes that no key gives, from the shapes of a file's tensors (name -> shape)."""
        layers = list(self.layers)
        for i, layer in enumerate(layers):
            if layer.gla is not None and layer.gla.decay_rank is None:
                shape = shapes.get(f"l{i}.mix.a1")
                if shape is None or len(shape) != 2:
                    raise ConfigError(f"layers[{i}]: the file has no matrix 'l{i}.mix.a1' to say the decay's rank")
                layers[i] = replace(layer, gla=replace(layer.gla, decay_rank=int(shape[0])))
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "layers": [x.to_dict() for x in self.layers],
                             "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
        if self.bigram is not None:
            d["embedding"] = {"bigram": self.bigram.to_dict()}
        return copy.deepcopy(d)
