"""Typed configuration of the Nebanex decoder, read from its config.json keys.

A Nebanex config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, `embedding.scale`,
`logit_softcap` (absent or null: the logits are not capped) and `layers`: a list with one entry per layer, each with
`type` ('parallel': two mixers side by side), `mixer` (`left`: heads, kv_heads, dim, vdim, scale, bias_max and
q_temp.{coef, every}; `right`: heads, dim, vdim, tau) and `mlp` (null for no feed-forward, or kind 'moe' with
router.{experts, top}, expert.ff and shared.ff or no shared expert).  Every size and constant that can differ between two
models of the design is a key; sizes that no key names (the rows of the distance-bias table, the inner width of the
decay's projections) are those of the stored tensors.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .base import ConfigError, KeyReader


def _object(data: Mapping[str, Any], key: str, where: str, required: bool = True):
    v = data.get(key)
    if v is None:
        if required:
            raise ConfigError(f"{where}: required key '{key}' (an object) is missing")
        return None
    if not isinstance(v, Mapping):
        raise ConfigError(f"{where}: '{key}' must be an object{'' if required else ' or null'}")
    return v


@dataclass(frozen=True)
class BiasAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    growth_coef: float | None      # None: queries get no factor by position
    growth_every: int

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "BiasAttentionConfig":
        r = KeyReader(data, where)
        heads, kv_heads = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
        if heads % kv_heads:
            raise ConfigError(f"{where}: 'heads' ({heads}) must be a multiple of 'kv_heads' ({kv_heads})")
        coef, every = None, 0
        growth = _object(data, "q_temp", where, required=False)
        if growth is not None:
            g = KeyReader(growth, where + ".q_temp")
            coef, every = g.number("coef"), g.integer("every", minimum=1)
        return cls(heads, kv_heads, r.integer("dim", minimum=1), r.integer("vdim", minimum=1), r.number("scale"),
                   r.integer("bias_max", minimum=2), coef, every)


@dataclass(frozen=True)
class LinearAttentionConfig:
    heads: int
    dim: int
    vdim: int
    tau: float

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "LinearAttentionConfig":
        r = KeyReader(data, where)
        return cls(r.integer("heads", minimum=1), r.integer("dim", minimum=1), r.integer("vdim", minimum=1),
                   r.number("tau", positive=True))


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int | None          # None: no shared expert

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "ExpertsConfig":
        KeyReader(data, where).string("kind", check=lambda v: v == "moe")
        router = KeyReader(_object(data, "router", where), where + ".router")
        experts = router.integer("experts", minimum=1)
        top = router.integer("top", minimum=1)
        if top > experts:
            raise ConfigError(f"{where}.router: 'top' ({top}) is larger than 'experts' ({experts})")
        ff = KeyReader(_object(data, "expert", where), where + ".expert").integer("ff", minimum=1)
        shared = _object(data, "shared", where, required=False)
        shared_ff = None if shared is None else KeyReader(shared, where + ".shared").integer("ff", minimum=1)
        return cls(experts, top, ff, shared_ff)


@dataclass(frozen=True)
class NebanexLayer:
    left: BiasAttentionConfig
    right: LinearAttentionConfig
    mlp: ExpertsConfig | None


@dataclass(frozen=True)
class NebanexConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    logit_softcap: float | None
    layers: tuple[NebanexLayer, ...]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str = "config.json") -> "NebanexConfig":
        r = KeyReader(data, where)
        architecture = r.string("architecture")
        eps = KeyReader(_object(data, "norm", where), where + ".norm").number("eps", positive=True)
        scale = KeyReader(_object(data, "embedding", where), where + ".embedding").number("scale")
        cap = r.number("logit_softcap", None, positive=True)
        raw = data.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError(f"{where}: required key 'layers' (a list of layers) is missing or empty")
        layers = []
        for i, entry in enumerate(raw):
            at = f"{where}.layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at}: must be an object")
            KeyReader(entry, at).string("type", check=lambda v: v == "parallel")
            mixer = _object(entry, "mixer", at)
            left = BiasAttentionConfig.from_dict(_object(mixer, "left", at + ".mixer"), at + ".mixer.left")
            right = LinearAttentionConfig.from_dict(_object(mixer, "right", at + ".mixer"), at + ".mixer.right")
            mlp = _object(entry, "mlp", at, required=False)
            layers.append(NebanexLayer(left, right, None if mlp is None else ExpertsConfig.from_dict(mlp, at + ".mlp")))
        return cls(architecture, r.integer("vocab", minimum=1), r.integer("width", minimum=1), eps, scale, cap, tuple(layers))
