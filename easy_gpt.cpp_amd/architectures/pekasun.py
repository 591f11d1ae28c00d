"""Pekasun decoder: typed configuration -> ModelSpec.

Tensor names: `embed`, `embed.norm`, `l<i>.norm1`, `l<i>.mix.*`, `l<i>.mlp.{gate,up,down}`, `final.norm`, `head`.
A layer is the parallel arrangement (one norm, mixer and feed-forward both read it, both are added); norms have one
gain for all coordinates.  An entry of the configuration's layer list that names `weights_of: j` becomes a second
run of layer j with a cache of its own, so the list of layers holds only those with tensors.
"""
from __future__ import annotations

from ..config.pekasun import LayerConfig, PekasunConfig
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

MAX_POSITION = 2**31 - 2        # the design names no longest sequence: positions are 32-bit integers


def _mixer_spec(layer: LayerConfig, prefix: str, eps: float) -> PartSpec:
    m = layer.mixer
    if m.kind == "attention":
        return PartSpec(
            "normed_attention",
            dict(n_heads=m.heads, n_kv_heads=m.kv_heads, key_dim=m.dim, value_dim=m.vdim, scale=m.scale, window=m.window,
                 keep_first=m.keep_first, eps=eps, norm_values=True,
                 names=dict(q="q", k="k", v="v", o="o", q_norm="q.norm", k_norm="k.norm")),
            prefix=prefix,
        )
    rot = m.rotation
    position = PartSpec("none", {})
    if rot is not None and rot.dims > 0:
        scaling = None if rot.factor is None else dict(factor=rot.factor, original=rot.original, fast=rot.fast, slow=rot.slow)
        position = PartSpec("rope_interleaved", dict(theta=rot.base, rotary_dim=rot.dims, scaling=scaling))
    return PartSpec(
        "latent_attention",
        dict(n_heads=m.heads, plain_dim=m.dim, rotated_dim=m.rot_dim, value_dim=m.vdim, latent_dim=m.kv_rank, scale=m.scale,
             window=m.window, keep_first=m.keep_first, eps=eps, sink=True, gated=True, position=position,
             names=dict(q="q", down="dkv", down_norm="dkv.norm", up_k="uk", up_v="uv", sink="sink", gate="g", o="o")),
        prefix=prefix,
    )


def pekasun_spec(cfg: PekasunConfig) -> ModelSpec:
    layers, index_of = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}."
        index_of[i] = len(layers)
        layers.append(
            LayerSpec(
                block="parallel" if layer.ff is not None else "parallel_mixer_only",
                mixer=_mixer_spec(layer, p + "mix.", cfg.eps),
                feed_forward=None if layer.ff is None else PartSpec(
                    "swiglu", dict(intermediate_size=layer.ff, names=("gate", "up", "down"), unrounded=True), prefix=p + "mlp."),
                norms={"input": PartSpec("rmsnorm_scalar", dict(eps=cfg.eps, name="norm1"), prefix=p)},
            )
        )
    run_order = tuple(
        RunSpec(layer=index_of[i if layer.weights_of is None else layer.weights_of], cache=i)
        for i, layer in enumerate(cfg.layers)
    )
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=MAX_POSITION,
        embedding=PartSpec("token_embedding_normed", dict(eps=cfg.eps, name="embed", norm_name="embed.norm"), prefix=""),
        layers=tuple(layers),
        run_order=run_order,
        final_norm=PartSpec("rmsnorm_scalar", dict(eps=cfg.eps, name="final.norm"), prefix=""),
        output_head=PartSpec("linear_head", dict(tied=False, name="head"), prefix=""),
    )


PEKASUN = register_architecture(
    Architecture(name="Pekasun", config_class=PekasunConfig, build_spec=pekasun_spec, model_types=("pekasun",)),
    replace=True,
)
