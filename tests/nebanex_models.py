"""Small Nebanex configurations and weights for the tests: sizes that differ in every respect, weights drawn so that
activations are of order one, attention is peaked, the distance bias is strong and the state's decays are neither 0
nor 1 (with weights of N(0, 0.02) a key that is wrongly seen, a bias from the wrong bucket or a lost state would
hardly move the logits).  The routed experts' outputs are small beside the stream: a float32 comparison (3e-5)
still sees every fault of the routing, while a choice between two experts whose logits nearly tie, which bfloat16
rounding of the router's input may turn, stays below the bfloat16 tolerance.  The tensor names are written out here,
not taken from the engine."""
from __future__ import annotations

import json
import os

import torch

from easy_gpt.cpp_amd.weights import write_safetensors


def left(heads, kv_heads, dim, vdim, scale, bias_max, coef=0.4, every=16):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max}
    if every:
        m["q_temp"] = {"coef": coef, "every": every}
    return m


def right(heads, dim, vdim, tau):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}


def moe(experts, top, ff, shared_ff):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff}
    return m


def layer(l, r, mlp):
    return {"type": "parallel", "mixer": {"left": l, "right": r}, "mlp": mlp}


# sizes that are of no kernel's liking: two layers of different sizes, a bias table of 8 rows whose last row starts at 20
CONFIG_A = {
    "architecture": "Nebanex", "vocab": 300, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 3.0},
    "logit_softcap": 8.0,
    "layers": [
        layer(left(4, 2, 16, 24, 0.25, 20, 0.5, 16), right(2, 16, 24, 4.0), moe(6, 2, 48, 64)),
        layer(left(2, 1, 32, 16, 0.2, 33, 0.25, 7), right(4, 8, 16, 16.0), moe(4, 3, 40, 32)),
    ],
}
# multiples of nothing: a width of 100, heads of 12 and 20, one query head per key/value head, one expert per token, no shared
# expert, a layer without a feed-forward, a query factor that changes at every position and a layer without one, tau 1,
# no cap on the logits
CONFIG_B = {
    "architecture": "Nebanex", "vocab": 257, "width": 100, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
    "layers": [
        layer(left(3, 3, 12, 20, 0.3, 9, 0.2, 1), right(3, 10, 12, 1.0), moe(5, 1, 50, None)),
        layer(left(1, 1, 20, 12, -0.25, 40, 0, 0), right(1, 36, 70, 2.0), None),
        layer(left(5, 1, 8, 8, 0.35, 12, 1.0, 3), right(2, 6, 100, 8.0), moe(3, 3, 30, 20)),
    ],
}
# multiples of 16, so that the matrix-core attention runs; every expert chosen; keys of 64 and 160 in the state
CONFIG_C = {
    "architecture": "Nebanex", "vocab": 411, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 10.0},
    "logit_softcap": 25.0,
    "layers": [
        layer(left(4, 1, 64, 32, 0.11, 50, 0.35, 64), right(2, 64, 80, 4.0), moe(8, 8, 64, 32)),
        layer(left(8, 2, 32, 64, 0.18, 100, 0.2, 96), right(1, 160, 64, 12.0), moe(16, 4, 32, 96)),
    ],
}
CONFIGS = {"A": (CONFIG_A, 5, 8, 5), "B": (CONFIG_B, 6, 6, 3), "C": (CONFIG_C, 7, 12, 8)}      # config, seed, bias rows, decay rank


def draw_weights(cfg: dict, seed: int, bias_rows: int = 8, rank: int = 5, sharp: float = 3.0) -> dict[str, torch.Tensor]:
    """name -> float32 tensor whose values are bfloat16 numbers (so that both precisions load the same model)."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]
    s = cfg["embedding"]["scale"]

    def matrix(out_f, in_f, gain=1.0):
        return torch.randn(out_f, in_f, generator=g) * (gain / in_f ** 0.5)

    def gains(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    def small(n, size=0.3):
        return size * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], width, generator=g) / s, "final.norm": gains(width), "final.norm.b": small(width),
         "head": matrix(cfg["vocab"], width, 2.0)}
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        w[p + "norm1"], w[p + "norm1.b"] = gains(width), small(width)
        l, r = entry["mixer"]["left"], entry["mixer"]["right"]
        q = p + "mix.left."
        hq, hk, dk, dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
        w[q + "q"], w[q + "q.b"] = matrix(hq * dk, width), small(hq * dk)
        w[q + "k"], w[q + "k.b"] = matrix(hk * dk, width), small(hk * dk)
        w[q + "v"], w[q + "v.b"] = matrix(hk * dv, width), small(hk * dv)
        w[q + "q.norm"], w[q + "k.norm"] = gains(hq * dk) * sharp, gains(hk * dk)
        w[q + "rel"] = 2.0 * torch.randn(bias_rows, hq, generator=g)
        w[q + "g"] = matrix(hq * dv, width, 2.0)
        w[q + "o"], w[q + "o.b"] = matrix(width, hq * dv), small(width)
        q = p + "mix.right."
        hr, dk, dv = r["heads"], r["dim"], r["vdim"]
        w[q + "q"], w[q + "k"] = matrix(hr * dk, width, 2.0), matrix(hr * dk, width)
        w[q + "v"], w[q + "g"] = matrix(hr * dv, width), matrix(hr * dv, width, 2.0)
        w[q + "o"], w[q + "norm"] = matrix(width, hr * dv), gains(dv)
        w[q + "a1"], w[q + "a2"] = matrix(rank, width), matrix(hr * dk, rank, 1.5)
        w[q + "a2.b"] = 1.5 + torch.randn(hr * dk, generator=g)
        w[p + "mix.left.out"], w[p + "mix.right.out"] = gains(width), gains(width) * 0.7
        mlp = entry.get("mlp")
        if mlp:
            w[p + "norm2"], w[p + "norm2.b"] = gains(width), small(width)
            q = p + "mlp."
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                w[f"{q}e{e}.gate"], w[f"{q}e{e}.up"] = matrix(ff, width), matrix(ff, width)
                w[f"{q}e{e}.down"] = matrix(width, ff, 0.05)
            w[q + "router"], w[q + "router.b"] = matrix(mlp["router"]["experts"], width, 4.0), small(mlp["router"]["experts"], 1.0)
            if mlp.get("shared"):
                f2 = mlp["shared"]["ff"]
                w[q + "shared.gate"], w[q + "shared.up"], w[q + "shared.down"] = matrix(f2, width), matrix(f2, width), matrix(width, f2, 0.7)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(model_dir: str, cfg: dict, seed: int, bias_rows: int = 8, rank: int = 5, change=None) -> str:
    """Writes config.json and model.safetensors (bfloat16); `change(weights)` may edit the drawn tensors first."""
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    w = draw_weights(cfg, seed, bias_rows, rank)
    if change is not None:
        change(w)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in w.items()})
    return model_dir
