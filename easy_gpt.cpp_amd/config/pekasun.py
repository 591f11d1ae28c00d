"""Typed configuration of the Pekasun decoder, read from its config.json keys.

A Pekasun config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps` and `layers`: a list
with one entry per layer run, each with `type` (which mixer: 'attention' or 'latent_attention'), `mixer` (that
mixer's sizes and constants), `mlp` (`{"kind": "dense", "ff": n}` or null for no feed-forward) and optionally
`weights_of: j` (the entry runs with the tensors of layer j and a cache of its own).  Every size and constant that
can differ between two models of the design is a key; nothing here is a default that hides a missing key, except
where the design says that a key may be absent (a mask without `keep_first`, a rotation without `scaling`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class RotationConfig:
    """Rotary positions on the first `dims` places of a rotated part; `scaling` None or (factor, original, fast, slow)."""

    base: float
    dims: int
    factor: float | None = None
    original: float | None = None
    fast: float | None = None
    slow: float | None = None

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str) -> "RotationConfig":
        r = KeyReader(data, where)
        base = r.number("base", positive=True)
        dims = r.integer("dims", minimum=0)
        if dims % 2:
            raise ConfigError(f"{where}: 'dims' ({dims}) must be even: places are rotated in pairs")
        sc = data.get("scaling")
        if sc is None:
            return cls(base, dims)
        if not isinstance(sc, Mapping):
            raise ConfigError(f"{where}: 'scaling' must be an object or null")
        s = KeyReader(sc, where + ".scaling")
        return cls(base, dims, s.number("factor", positive=True), s.number("original", positive=True),
                   s.number("fast", positive=True), s.number("slow", positive=True))


@dataclass(frozen=True)
class MixerConfig:
    """Sizes and constants of one mixer.  kind 'attention': heads, kv_heads, dim, vdim, scale, window, keep_first.
    kind 'latent_attention': heads, dim, rot_dim, vdim, kv_rank, scale, window, keep_first, rotation."""

    kind: str
    heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None
    keep_first: int = 0
    kv_heads: int = 0
    rot_dim: int = 0
    kv_rank: int = 0
    rotation: RotationConfig | None = None

    @classmethod
    def from_dict(cls, kind: str, data: Mapping[str, Any], where: str) -> "MixerConfig":
        r = KeyReader(data, where)
        heads = r.integer("heads", minimum=1)
        dim = r.integer("dim", minimum=1)
        vdim = r.integer("vdim", minimum=1)
        scale = r.number("scale")
        mask = data.get("mask")
        window, keep_first = None, 0
        if mask is not None:
            if not isinstance(mask, Mapping):
                raise ConfigError(f"{where}: 'mask' must be an object or null")
            m = KeyReader(mask, where + ".mask")
            window = m.integer("size", None, minimum=1)
            keep_first = m.integer("keep_first", 0, minimum=0)
        if kind == "attention":
            kv_heads = r.integer("kv_heads", minimum=1)
            if heads % kv_heads:
                raise ConfigError(f"{where}: 'heads' ({heads}) must be a multiple of 'kv_heads' ({kv_heads})")
            return cls(kind, heads, dim, vdim, scale, window, keep_first, kv_heads=kv_heads)
        if kind == "latent_attention":
            rot_dim = r.integer("rot_dim", minimum=0)
            rank = r.integer("kv_rank", minimum=1)
            rotation = None
            if data.get("rot") is not None:
                if not isinstance(data["rot"], Mapping):
                    raise ConfigError(f"{where}: 'rot' must be an object or null")
                rotation = RotationConfig.from_dict(data["rot"], where + ".rot")
                if rotation.dims > rot_dim:
                    raise ConfigError(f"{where}: rot.dims ({rotation.dims}) is larger than rot_dim ({rot_dim})")
            return cls(kind, heads, dim, vdim, scale, window, keep_first, rot_dim=rot_dim, kv_rank=rank, rotation=rotation)
        raise ConfigError(f"{where}: unknown layer type '{kind}' (known: attention, latent_attention)")


@dataclass(frozen=True)
class LayerConfig:
    mixer: MixerConfig
    ff: int | None             # inner width of the dense feed-forward, None: the layer has none
    weights_of: int | None     # the layer whose tensors this entry uses, None: its own


@dataclass(frozen=True)
class PekasunConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    layers: tuple[LayerConfig, ...]

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], where: str = "config.json") -> "PekasunConfig":
        r = KeyReader(data, where)
        architecture = r.string("architecture")
        norm = data.get("norm")
        if not isinstance(norm, Mapping):
            raise ConfigError(f"{where}: required key 'norm' (an object with 'eps') is missing")
        eps = KeyReader(norm, where + ".norm").number("eps", positive=True)
        raw = data.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError(f"{where}: required key 'layers' (a list of layers) is missing or empty")
        layers = []
        for i, entry in enumerate(raw):
            at = f"{where}.layers[{i}]"
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{at}: must be an object")
            e = KeyReader(entry, at)
            kind = e.string("type")
            if not isinstance(entry.get("mixer"), Mapping):
                raise ConfigError(f"{at}: required key 'mixer' is missing")
            mixer = MixerConfig.from_dict(kind, entry["mixer"], at + ".mixer")
            ff = None
            if entry.get("mlp") is not None:
                if not isinstance(entry["mlp"], Mapping):
                    raise ConfigError(f"{at}: 'mlp' must be an object or null")
                m = KeyReader(entry["mlp"], at + ".mlp")
                m.string("kind", check=lambda v: v == "dense")
                ff = m.integer("ff", minimum=1)
            src = e.integer("weights_of", None, minimum=0)
            layers.append(LayerConfig(mixer, ff, src))
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is None:
                continue
            at = f"{where}.layers[{i}]"
            if j >= len(layers) or j == i or layers[j].weights_of is not None:
                raise ConfigError(f"{at}: 'weights_of' ({j}) must name another layer that has tensors of its own")
            if (layers[j].mixer, layers[j].ff) != (layer.mixer, layer.ff):
                raise ConfigError(f"{at}: a layer that uses layer {j}'s weights must have layer {j}'s sizes")
        return cls(architecture, r.integer("vocab", minimum=1), r.integer("width", minimum=1), eps, tuple(layers))
