"""Typed configuration of the Vafodra decoder.

config.json names the design in `architecture` and gives every size: `vocab`, `width`, `embedding.scale`,
`norm.eps`, `residual_mult`, and `layers`, a list with one entry a layer: `type` ("parallel": attention and a
state-space layer side by side; "delta": the gated delta rule), `mixer` (the sizes of that type), `mlp`
(`{"kind": "dense", "ff": n}` or null) and optionally `weights_of`, the index of the layer whose tensors this
one runs with.  Every error names its key.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig, coerce


_REQUIRED = object()


def _get(d: Dict[str, Any], key: str, where: str, kind=int, least=None, default=_REQUIRED):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        if default is not _REQUIRED and isinstance(d, dict):
            return default  # what config.json does not mention, the model does not have
        raise ConfigError(f"config.json: required key '{where}.{key}' is missing")
    try:
        v = coerce(d[key], f"{where}.{key}", kind)
    except ConfigError:
        raise
    if least is not None and v < least:
        raise ConfigError(f"config.json: '{where}.{key}' must be at least {least}, found {v}")
    return v


@dataclass(frozen=True)
class AttentionSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int

    @classmethod
    def from_dict(cls, d, where):
        mask = d.get("mask") if isinstance(d, dict) else None
        if not isinstance(mask, dict):
            raise ConfigError(f"config.json: required key '{where}.mask' is missing")
        heads = _get(d, "heads", where, least=1)
        dim = _get(d, "dim", where, least=1)
        c = cls(heads, _get(d, "kv_heads", where, least=1, default=heads), dim, _get(d, "vdim", where, least=1, default=dim),
                _get(d, "scale", where, float), _get(mask, "size", where + ".mask", least=1),
                _get(mask, "keep_first", where + ".mask", least=0, default=0))
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of kv_heads ({c.kv_heads})")
        return c

    def to_dict(self):
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "mask": {"keep_first": self.keep_first, "size": self.window}, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class StateSpaceSide:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, d, where):
        c = cls(_get(d, "heads", where, least=1), _get(d, "vdim", where, least=1), _get(d, "state", where, least=1),
                _get(d, "groups", where, least=1, default=1), _get(d, "conv", where, least=1),
                _get(d, "norm_groups", where, least=1, default=1))
        if c.heads % c.groups:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of groups ({c.groups})")
        if (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"config.json: '{where}.norm_groups' ({c.norm_groups}) does not divide heads * vdim")
        return c

    def to_dict(self):
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class DeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @classmethod
    def from_dict(cls, d, where):
        heads = _get(d, "heads", where, least=1)
        dim = _get(d, "dim", where, least=1)
        c = cls(heads, _get(d, "kv_heads", where, least=1, default=heads), dim, _get(d, "vdim", where, least=1, default=dim),
                _get(d, "conv", where, least=1))
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of kv_heads ({c.kv_heads})")
        return c

    def to_dict(self):
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class VafodraLayer:
    type: str  # "parallel" | "delta"
    left: Optional[AttentionSide]
    right: Optional[StateSpaceSide]
    delta: Optional[DeltaMixer]
    ff: Optional[int]  # None: no feed-forward
    weights_of: Optional[int]

    @classmethod
    def from_dict(cls, d, i: int):
        where = f"layers[{i}]"
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        kind = d.get("type")
        mixer = d.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"config.json: required key '{where}.mixer' is missing")
        left = right = delta = None
        if kind == "parallel":
            left = AttentionSide.from_dict(mixer.get("left"), where + ".mixer.left")
            right = StateSpaceSide.from_dict(mixer.get("right"), where + ".mixer.right")
        elif kind == "delta":
            delta = DeltaMixer.from_dict(mixer, where + ".mixer")
        else:
            raise ConfigError(f"config.json: '{where}.type' must be 'parallel' or 'delta', found {kind!r}")
        mlp, ff = d.get("mlp"), None
        if mlp is not None:
            if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                raise ConfigError(f"config.json: '{where}.mlp.kind' must be 'dense' (or mlp null)")
            ff = _get(mlp, "ff", where + ".mlp", least=1)
        weights_of = d.get("weights_of")
        if weights_of is not None:
            weights_of = coerce(weights_of, where + ".weights_of", int)
        return cls(kind, left, right, delta, ff, weights_of)

    def same_shape(self, other: "VafodraLayer") -> bool:
        return (self.type, self.left, self.right, self.delta, self.ff) == \
            (other.type, other.left, other.right, other.delta, other.ff)

    def to_dict(self):
        d: Dict[str, Any] = {"type": self.type}
        d["mixer"] = {"left": self.left.to_dict(), "right": self.right.to_dict()} if self.type == "parallel" \
            else self.delta.to_dict()
        d["mlp"] = None if self.ff is None else {"ff": self.ff, "kind": "dense"}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class VafodraConfig(ModelConfig):
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    residual_mult: float
    layers: Tuple[VafodraLayer, ...]
    architecture: str = "Vafodra"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "VafodraConfig":
        top = "config"
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(VafodraLayer.from_dict(x, i) for i, x in enumerate(layers))
        for i, layer in enumerate(parsed):
            j = layer.weights_of
            if j is None:
                continue
            if not 0 <= j < len(parsed) or j == i or parsed[j].weights_of is not None:
                raise ConfigError(f"config.json: 'layers[{i}].weights_of' must name another layer with tensors of its own")
            if not layer.same_shape(parsed[j]):
                raise ConfigError(f"config.json: 'layers[{i}]' runs with the weights of layer {j} but differs from it")
        if not isinstance(d.get("embedding"), dict) or not isinstance(d.get("norm"), dict):
            raise ConfigError("config.json: 'embedding' and 'norm' must be objects")
        return cls(vocab=_get(d, "vocab", top, least=1), width=_get(d, "width", top, least=1),
                   embedding_scale=_get(d["embedding"], "scale", "embedding", float),
                   norm_eps=_get(d["norm"], "eps", "norm", float),
                   residual_mult=_get(d, "residual_mult", top, float), layers=parsed,
                   architecture=str(d.get("architecture", "Vafodra")))

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy({
            "architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
            "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
            "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width})
