"""A plain, slow Pekasun decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.

It shares no code with the engine: it reads a model folder with its own few lines and knows the tensor names
itself.  Notation: x [T, W] is the residual stream of one sequence, positions count from 0, a linear weight is
[out, in] and applied as x W^T.

The design: x = N(embed[token]) with a scalar-gain RMS norm; every layer is parallel, h = N1(x),
x <- x + mixer(h) + ff(h); two kinds of mixer (grouped-query attention with normed queries, keys and values and a
window that keeps the first tokens; latent attention with a shared rotated key part, a window, a sink in the
softmax and an output gate); a gated feed-forward; a last scalar-gain norm and the output matrix.  A layer may
run with another layer's weights (`weights_of`).
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np
import torch

F64 = torch.float64


def read_safetensors(path: str) -> dict[str, torch.Tensor]:
    with open(path, "rb") as f:
        raw = f.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8 : 8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        buf = raw[base + b : base + e]
        if info["dtype"] == "F32":
            a = torch.from_numpy(np.frombuffer(buf, dtype="<f4").copy())
        elif info["dtype"] == "BF16":
            u16 = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            a = torch.from_numpy(u16.view(np.float32).copy())
        else:
            raise ValueError(info["dtype"])
        out[name] = a.reshape(info["shape"]).to(F64)
    return out


def read_model(model_dir: str, round_to_bf16: bool = False):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = read_safetensors(os.path.join(model_dir, "model.safetensors"))
    if round_to_bf16:
        w = {k: v.to(torch.float32).to(torch.bfloat16).to(F64) for k, v in w.items()}
    return cfg, w


# ----------------------------------------------------------------------------- mechanisms
def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, gain, eps):
    """RMS norm with one gain for all coordinates."""
    return unit_rms(x, eps) * gain.reshape(())


def vector_norm(x, weight, eps):
    """RMS norm over the last axis with a weight per coordinate (plain weight, not one-plus)."""
    return unit_rms(x, eps) * weight


def gated_feed_forward(h, gate, up, down):
    g = h @ gate.T
    return ((g * torch.sigmoid(g)) * (h @ up.T)) @ down.T


def visible_window_keep_first(n, size, keep_first):
    """[n, n] bool: query i sees key j if j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(n).reshape(n, 1)
    j = torch.arange(n).reshape(1, n)
    return (j <= i) & ((i - j < size) | (j < keep_first))


def softmax_with_sink(scores, visible, sink=None):
    """Softmax over the visible keys of every row of scores [..., n, n]; with `sink` [heads] the denominator also
    holds exp(sink_h), which has no key and no value.  scores [heads, n, n]."""
    s = scores.masked_fill(~visible, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.reshape(-1, 1, 1))
    e = torch.exp(s - m)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink.reshape(-1, 1, 1) - m)
    return e / denom


def yarn_frequencies(rot):
    """(frequencies [dims / 2], factor on cos and sin) of a rotation description {base, dims, scaling}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, freqs, mag):
    """x [..., n, d]: the pairs (2i, 2i + 1) of the first 2 * len(freqs) coordinates are rotated by
    positions[n] * freqs[i]; cos and sin are multiplied by `mag`; the rest passes unchanged."""
    d = 2 * freqs.shape[0]
    a = positions.to(F64).reshape(-1, 1) * freqs.reshape(1, -1)
    c, s = torch.cos(a) * mag, torch.sin(a) * mag
    u, v = x[..., 0:d:2], x[..., 1:d:2]
    out = x.clone()
    out[..., 0:d:2] = u * c - v * s
    out[..., 1:d:2] = v * c + u * s
    return out


def normed_attention(h, w, p, m, eps):
    """Grouped-query attention without positions: queries and keys normed per head with a shared weight, values
    divided by their root mean square, window with kept first tokens."""
    n = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[p + "q"].T).reshape(n, H, dk)
    k = (h @ w[p + "k"].T).reshape(n, G, dk)
    v = (h @ w[p + "v"].T).reshape(n, G, dv)
    q = vector_norm(q, w[p + "q.norm"], eps)
    k = vector_norm(k, w[p + "k.norm"], eps)
    v = unit_rms(v, eps)
    rep = H // G
    kh = k.repeat_interleave(rep, dim=1)
    vh = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, kh) * float(m["scale"])
    mask = m.get("mask") or {}
    vis = visible_window_keep_first(n, int(mask.get("size", 1 << 60)), int(mask.get("keep_first", 0)))
    pr = softmax_with_sink(scores, vis)
    o = torch.einsum("hij,jhd->ihd", pr, vh).reshape(n, H * dv)
    return o @ w[p + "o"].T


def latent_attention(h, w, p, m, eps):
    """Latent attention: a normed latent c per token from which every head's unrotated key and value are made, one
    rotated key part shared by the heads, a window, a sink per head in the softmax, a sigmoid gate on the output."""
    n = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(n)
    q = (h @ w[p + "q"].T).reshape(n, H, d + r)
    dkv = h @ w[p + "dkv"].T
    c = vector_norm(dkv[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = dkv[:, rank:]
    freqs, mag = yarn_frequencies(m["rot"]) if m.get("rot") else (torch.zeros(0, dtype=F64), 1.0)
    q_un, q_rot = q[..., :d], q[..., d:]
    q_rot = rotate_interleaved(q_rot.transpose(0, 1), pos, freqs, mag).transpose(0, 1)
    k_rot = rotate_interleaved(k_rot, pos, freqs, mag)
    k_un = (c @ w[p + "uk"].T).reshape(n, H, d)
    v = (c @ w[p + "uv"].T).reshape(n, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_un, k_un) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * float(m["scale"])
    mask = m.get("mask") or {}
    vis = visible_window_keep_first(n, int(mask.get("size", 1 << 60)), int(mask.get("keep_first", 0)))
    pr = softmax_with_sink(scores, vis, w[p + "sink"])
    o = torch.einsum("hij,jhd->ihd", pr, v).reshape(n, H * dv)
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


MIXERS = {"attention": normed_attention, "latent_attention": latent_attention}


def forward(cfg, w, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer run, if asked)."""
    eps = float(cfg["norm"]["eps"])
    x = scalar_norm(w["embed"][torch.as_tensor(tokens, dtype=torch.long)], w["embed.norm"], eps)
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        h = scalar_norm(x, w[p + "norm1"], eps)
        delta = MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp"):
            delta = delta + gated_feed_forward(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
        x = x + delta
        streams.append(x)
    logits = scalar_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(streams)) if return_layers else logits
