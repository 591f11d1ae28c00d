"""Small Pekasun configurations and weights for the tests: sizes that differ in every respect, weights drawn so that
activations are of order one and attention is peaked (with weights of N(0, 0.02) every key would get nearly the
same weight, and a key that is wrongly seen or missed would hardly move the logits).  The tensor names are written
out here, not taken from the engine."""
from __future__ import annotations

import json
import os

import torch

from easy_gpt.cpp_amd.weights import write_safetensors


def latent(heads, dim, rot_dim, vdim, rank, window, scale, base=10000.0, dims=None, scaling=None, keep_first=None):
    rot = None if rot_dim == 0 else {"base": base, "dims": rot_dim if dims is None else dims, "scaling": scaling}
    if rot is not None and scaling is None:
        del rot["scaling"]
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}
    if window:
        m["mask"] = {"size": window} if keep_first is None else {"size": window, "keep_first": keep_first}
    return {"type": "latent_attention", "mixer": m}


def attention(heads, kv_heads, dim, vdim, window, keep_first, scale):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first} if keep_first is not None else {"size": window}
    return {"type": "attention", "mixer": m}


def layer(entry, ff, weights_of=None):
    out = dict(entry, mlp=None if ff is None else {"kind": "dense", "ff": ff})
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}

# two latent layers and two attention layers, the second of each kind on the first one's weights
CONFIG_A = {
    "architecture": "Pekasun", "vocab": 300, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        layer(latent(2, 16, 8, 24, 40, 20, 0.2, scaling=YARN), 96),
        layer(attention(4, 2, 16, 32, 12, 3, 0.5), 96),
        layer(latent(2, 16, 8, 24, 40, 20, 0.2, scaling=YARN), 96, weights_of=0),
        layer(attention(4, 2, 16, 32, 12, 3, 0.5), 96, weights_of=1),
    ],
}
# one query head per key/value head, a window that keeps one token and one that keeps none, a latent layer with one
# head whose rotated part is wider than its plain part and is rotated only in its first places, a layer without a
# feed-forward, a window of one token, a window wider than any test sequence
CONFIG_B = {
    "architecture": "Pekasun", "vocab": 257, "width": 96, "norm": {"eps": 1e-5},
    "layers": [
        layer(attention(3, 3, 32, 16, 7, 1, 0.3), 80),
        layer(latent(1, 8, 16, 8, 24, 33, 0.35, base=500.0, dims=12), None),
        layer(attention(2, 1, 16, 48, 1, 0, 0.4), 112),
        layer(latent(3, 16, 4, 16, 32, 4096, 0.25, base=100000.0, scaling={"factor": 8.0, "original": 16, "fast": 4.0, "slow": 1.0}), 64),
        layer(attention(2, 2, 48, 16, 5, 9, 0.2), 80),
    ],
}
# head sizes in multiples of 16 with a page-sized window, more kept tokens than a page holds, no mask at all on one layer
CONFIG_C = {
    "architecture": "Pekasun", "vocab": 411, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        layer(latent(4, 32, 16, 32, 48, 16, 0.15, base=20000.0), 160),
        layer(attention(4, 1, 64, 32, 32, 21, 0.25), 160),
        layer(attention(2, 2, 32, 64, None, None, 0.3), 160),
        layer(latent(4, 32, 16, 32, 48, 16, 0.15, base=20000.0), 160, weights_of=0),
    ],
}
# sizes that are multiples of nothing: a width of 100, heads of 12 and 20, a latent of 36 with an odd rotated part of 7
# (six places rotated), an inner width of 50, a latent window that keeps two tokens
CONFIG_E = {
    "architecture": "Pekasun", "vocab": 333, "width": 100, "norm": {"eps": 1e-6},
    "layers": [
        layer(latent(3, 12, 7, 20, 36, 9, 0.3, base=3000.0, dims=6, keep_first=2), 50),
        layer(attention(3, 1, 12, 20, 11, 2, 0.35), 50),
        layer(attention(5, 5, 20, 12, 6, 0, -0.3), None),
    ],
}
# latent layers without a rotated part (no positions enter at all), one on the other's weights
CONFIG_F = {
    "architecture": "Pekasun", "vocab": 99, "width": 48, "norm": {"eps": 1e-6},
    "layers": [layer(latent(2, 8, 0, 8, 16, 5, 0.3), 32), layer(latent(2, 8, 0, 8, 16, 5, 0.3), 32, weights_of=0)],
}
CONFIGS = {"A": (CONFIG_A, 5), "B": (CONFIG_B, 6), "C": (CONFIG_C, 7), "E": (CONFIG_E, 9), "F": (CONFIG_F, 10)}


def draw_weights(cfg: dict, seed: int, sharp: float = 3.0) -> dict[str, torch.Tensor]:
    """name -> float32 tensor whose values are bfloat16 numbers (so that both precisions load the same model)."""
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]

    def matrix(out_f, in_f, gain=1.0):
        return torch.randn(out_f, in_f, generator=g) * (gain / in_f ** 0.5)

    def gains(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    w = {"embed": torch.randn(cfg["vocab"], width, generator=g), "embed.norm": torch.tensor(1.3),
         "final.norm": torch.tensor(0.9), "head": matrix(cfg["vocab"], width, 2.0)}
    for i, entry in enumerate(cfg["layers"]):
        if "weights_of" in entry:
            continue
        p, m = f"l{i}.", entry["mixer"]
        w[p + "norm1"] = torch.tensor(1.0 + 0.1 * (i % 3))
        heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
        if entry["type"] == "attention":
            w[p + "mix.q"] = matrix(heads * dim, width)
            w[p + "mix.k"] = matrix(m["kv_heads"] * dim, width)
            w[p + "mix.v"] = matrix(m["kv_heads"] * vdim, width)
            w[p + "mix.q.norm"] = gains(dim) * sharp
            w[p + "mix.k.norm"] = gains(dim)
            w[p + "mix.o"] = matrix(width, heads * vdim, 0.5)
        else:
            rot, rank = m["rot_dim"], m["kv_rank"]
            w[p + "mix.q"] = matrix(heads * (dim + rot), width, sharp)
            w[p + "mix.dkv"] = matrix(rank + rot, width)
            w[p + "mix.dkv.norm"] = gains(rank)
            w[p + "mix.uk"] = matrix(heads * dim, rank)
            w[p + "mix.uv"] = matrix(heads * vdim, rank)
            w[p + "mix.sink"] = torch.randn(heads, generator=g) * 2.0
            w[p + "mix.g"] = matrix(heads * vdim, width, 2.0)
            w[p + "mix.o"] = matrix(width, heads * vdim, 0.5)
        if entry.get("mlp"):
            ff = entry["mlp"]["ff"]
            w[p + "mlp.gate"] = matrix(ff, width)
            w[p + "mlp.up"] = matrix(ff, width)
            w[p + "mlp.down"] = matrix(width, ff, 0.5)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in w.items()}


def write_model(model_dir: str, cfg: dict, seed: int, sharp: float = 3.0, change=None) -> str:
    """Writes config.json and model.safetensors (bfloat16, the scalars too); `change(weights)` may edit the drawn
    tensors before they are written."""
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    w = draw_weights(cfg, seed, sharp)
    if change is not None:
        change(w)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in w.items()})
    return model_dir
