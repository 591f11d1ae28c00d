"""A plain, slow Nebanex decoder: whole sequences, no cache, one function per mechanism, float64 on the CPU.

It shares no code with the engine: it reads a model folder with its own few lines and knows the tensor names
itself.  Notation: x [T, W] is the residual stream of one sequence, positions count from 0, a linear weight is
[out, in] and applied as x W^T.

The design: x = embed[token] * s; every layer is pre-norm with layer norms (weight and bias),
x <- x + mixer(LN1(x)), x <- x + ff(LN2(x)).  The mixer is two mixers side by side on the same input, each output
RMS-normed over the width, half their sum: on the left a grouped-query attention without rotation (biased
projections, queries and keys RMS-normed over the whole projection, a query factor that grows with the logarithm
of the position, a learned bias per head and distance bucket, a sigmoid output gate); on the right a gated linear
attention (a matrix state per head that decays per key channel).  The feed-forward is a mixture of experts with a
shared expert.  A last layer norm, the output matrix, and a tanh cap on the logits.
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


def read_model(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ----------------------------------------------------------------------------- mechanisms
def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def query_factor(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1) for every position p."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=F64)


def distance_bucket(n: int, rows: int, far: int) -> int:
    """The row of the bias table for distance n >= 0: the distance itself below rows // 2, then steps that grow
    with the logarithm of the distance and reach the last row at `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias(n_tokens, table, far):
    """[heads, T, T]: table[bucket(i - j), head] for j <= i (0 elsewhere)."""
    rows, heads = table.shape
    out = torch.zeros(heads, n_tokens, n_tokens, dtype=F64)
    per_distance = torch.stack([table[distance_bucket(n, rows, far)] for n in range(n_tokens)])      # [T, heads]
    for i in range(n_tokens):
        for j in range(i + 1):
            out[:, i, j] = per_distance[i - j]
    return out


def biased_attention(h, w, p, m, eps):
    """The left mixer on the normed input h [T, W]; w the tensors, p their prefix, m its sizes and constants."""
    t = h.shape[0]
    nq, nkv, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    q = rms_norm(q, w[p + "q.norm"], eps)                    # over the whole projection, all heads at once
    k = rms_norm(k, w[p + "k.norm"], eps)
    if m.get("q_temp") is not None:
        q = q * query_factor(range(t), m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    q, k, v = q.view(t, nq, dk), k.view(t, nkv, dk), v.view(t, nkv, dv)
    bias = distance_bias(t, w[p + "rel"], m["bias_max"])
    causal = torch.ones(t, t).tril().bool()
    heads = []
    for head in range(nq):
        g = head // (nq // nkv)
        s = (q[:, head] @ k[:, g].T) * m["scale"] + bias[head]
        s = s.masked_fill(~causal, -math.inf)
        heads.append(torch.softmax(s, dim=-1) @ v[:, g])
    o = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T + w[p + "o.b"]


def decayed_state_scan(q, k, v, alpha, state=None):
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  q, k, alpha [T, heads, dk]; v [T, heads,
    dv].  Returns o [T, heads, dv] and the last state [heads, dk, dv]."""
    t, nh, dk = q.shape
    dv = v.shape[-1]
    s = torch.zeros(nh, dk, dv, dtype=F64) if state is None else state.clone()
    out = torch.zeros(t, nh, dv, dtype=F64)
    for i in range(t):
        s = alpha[i][:, :, None] * s + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hkv,hk->hv", s, q[i])
    return out, s


def gated_linear_attention(h, w, p, m, eps):
    """The right mixer."""
    t = h.shape[0]
    nh, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T * dk ** -0.5).view(t, nh, dk)
    k = (h @ w[p + "k"].T).view(t, nh, dk)
    v = (h @ w[p + "v"].T).view(t, nh, dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(t, nh, dk)
    o, _ = decayed_state_scan(q, k, v, alpha)
    o = rms_norm(o, w[p + "norm"], eps).reshape(t, nh * dv)
    g = h @ w[p + "g"].T
    return (o * (g * torch.sigmoid(g))) @ w[p + "o"].T


def side_by_side(h, w, p, m, eps):
    left = biased_attention(h, w, p + "left.", m["left"], eps)
    right = gated_linear_attention(h, w, p + "right.", m["right"], eps)
    return 0.5 * (rms_norm(left, w[p + "left.out"], eps) + rms_norm(right, w[p + "right.out"], eps))


def gated_expert(h, w, p):
    g = h @ w[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, top):
    """Chosen experts [T, top] and their weights: softmax over the chosen logits only."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    idx = torch.argsort(-z, dim=-1, stable=True)[:, :top]          # the lower index among equal logits
    return idx, torch.softmax(torch.gather(z, -1, idx), dim=-1), z


def expert_mixture(h, w, p, mlp):
    idx, weight, _ = route(h, w, p, mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), weight[t]):
            out[t] += a * gated_expert(h[t : t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared") is not None:
        out = out + gated_expert(h, w, p + "shared.")
    return out


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


# ----------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, collect=None):
    """Logits [T, vocab] (float64) of one sequence; collect, if a list, gets the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        x = x + side_by_side(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + expert_mixture(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w, p + "mlp.", layer["mlp"])
        if collect is not None:
            collect.append(x.clone())
    z = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    return soft_cap(z, cap) if cap else z
