"""Nebanex decoder: typed configuration -> ModelSpec.

Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm1.b`, `l<i>.norm2`, `l<i>.norm2.b`, `l<i>.mix.{left,right}.*`,
`l<i>.mix.{left,right}.out`, `l<i>.mlp.{e<j>,shared}.{gate,up,down}`, `l<i>.mlp.router`, `l<i>.mlp.router.b`,
`final.norm`, `final.norm.b`, `head`.  A layer is the pre-norm arrangement with layer norms; its mixer is two mixers side
by side (softmax attention with a distance bias, and linear attention with a decaying state), its feed-forward a
mixture of experts with a shared expert.
"""
from __future__ import annotations

from ..config.nebanex import NebanexConfig, NebanexLayer
from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

MAX_POSITION = 2**31 - 2        # the design names no longest sequence: positions are 32-bit integers


def _norm(prefix: str, name: str, eps: float) -> PartSpec:
    return PartSpec("layernorm", dict(eps=eps, name=name, bias_name=name + ".b"), prefix=prefix)


def _layer_spec(layer: NebanexLayer, p: str, eps: float) -> LayerSpec:
    left, right = layer.left, layer.right
    growth = None if left.growth_coef is None else (left.growth_coef, left.growth_every)
    mixer = PartSpec(
        "side_by_side",
        dict(
            left=PartSpec("distance_bias_attention",
                          dict(n_heads=left.heads, n_kv_heads=left.kv_heads, key_dim=left.dim, value_dim=left.vdim,
                               scale=left.scale, eps=eps, bias_far=left.bias_max, query_growth=growth),
                          prefix=p + "mix.left."),
            right=PartSpec("gated_linear_attention",
                           dict(n_heads=right.heads, key_dim=right.dim, value_dim=right.vdim, tau=right.tau, eps=eps),
                           prefix=p + "mix.right."),
            eps=eps, factor=0.5, names=dict(left_out="left.out", right_out="right.out"),
        ),
        prefix=p + "mix.",
    )
    norms = {"mixer": _norm(p, "norm1", eps)}
    if layer.mlp is None:
        return LayerSpec(block="pre_norm_mixer_only", mixer=mixer, feed_forward=None, norms=norms)
    m = layer.mlp
    shared = None
    if m.shared_ff is not None:
        shared = PartSpec("swiglu", dict(intermediate_size=m.shared_ff, names=("gate", "up", "down"), unrounded=True),
                          prefix=p + "mlp.shared.")
    ff = PartSpec("expert_mixture", dict(n_experts=m.experts, top=m.top, intermediate_size=m.ff, shared=shared),
                  prefix=p + "mlp.")
    norms["feed_forward"] = _norm(p, "norm2", eps)
    return LayerSpec(block="pre_norm", mixer=mixer, feed_forward=ff, norms=norms)


def nebanex_spec(cfg: NebanexConfig) -> ModelSpec:
    layers = tuple(_layer_spec(layer, f"l{i}.", cfg.eps) for i, layer in enumerate(cfg.layers))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_position=MAX_POSITION,
        embedding=PartSpec("token_embedding_scaled", dict(scale=cfg.embedding_scale, name="embed"), prefix=""),
        layers=layers,
        run_order=tuple(RunSpec(layer=i, cache=i, state=i) for i in range(len(layers))),
        final_norm=_norm("", "final.norm", cfg.eps),
        output_head=PartSpec("linear_head", dict(tied=False, name="head", softcap=cfg.logit_softcap), prefix=""),
    )


NEBANEX = register_architecture(
    Architecture(name="Nebanex", config_class=NebanexConfig, build_spec=nebanex_spec, model_types=("nebanex",)),
    replace=True,
)
