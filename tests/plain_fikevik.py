"""A plain, slow implementation of the Fikevik decoder in float64: one function per mechanism, whole sequences only.

Nothing here is shared with the engine: no kernels, no cache, no parts. A model is a configuration (the dict that
config.json holds) and a dict of tensors by their names in the file. Every function takes the rows of one sequence,
positions 0, 1, 2, ... in order.

Notation: h [T, width] the rows a sublayer reads; weights are stored [out, in] and applied as h @ W.T.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def read_model_folder(folder):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {n: (t.to(F64) if t.is_floating_point() else t) for n, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def rms_norm(x, eps, weight=None):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, dim]: the pair (2i, 2i+1) of the first `dims` channels turns by positions * base^(-2i/dims)."""
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=F64)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(F64)[:, None] * freq[None, :]             # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def windowed_attention(h, w, pre, p, eps):
    """The left branch: grouped-query softmax attention over the last `mask.size` positions."""
    T = h.shape[0]
    H, G, D, V = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = (h @ w[pre + "v"].T).view(T, G, V)
    q = rms_norm(q, eps, w[pre + "q.norm"])
    k = rms_norm(k, eps, w[pre + "k.norm"])
    pos = torch.arange(T)
    q = rotate_pairs(q, pos, p["rot"]["dims"], p["rot"].get("base"))
    k = rotate_pairs(k, pos, p["rot"]["dims"], p["rot"].get("base"))
    v = rms_norm(v, eps)
    size = p["mask"]["size"]
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        lo = max(0, t - size + 1)
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:t + 1, g] @ q[t, hh]) * p["scale"] * w[pre + "temp"][hh]
            out[t, hh] = torch.softmax(s, dim=0) @ v[lo:t + 1, g]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def matrix_memory(h, w, pre, p, eps):
    """The right branch: a matrix memory per head with exponential input gate, kept stable by a running maximum."""
    T = h.shape[0]
    H, D, V, cap = p["heads"], p["dim"], p["vdim"], p["gate_cap"]
    q = (h @ w[pre + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, V)
    gi = cap * torch.tanh((h @ w[pre + "i"].T + w[pre + "i.b"]) / cap)                                   # [T, H]
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[pre + "f"].T + w[pre + "f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    m = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(gf[t] + m, gi[t])
        keep, take = torch.exp(gf[t] + m - m_new), torch.exp(gi[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    out = rms_norm(out, eps).reshape(T, H * V) * w[pre + "norm"]
    out = out * torch.sigmoid(h @ w[pre + "g"].T)
    return out @ w[pre + "o"].T


def gated_linear_attention(h, w, pre, p, eps):
    """The 'gla' mixer: a matrix state per head whose rows decay by a data-dependent factor per key channel."""
    T = h.shape[0]
    H, D, V, tau = p["heads"], p["dim"], p["vdim"], p["tau"]
    q = (h @ w[pre + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, V)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    decay = torch.exp(torch.nn.functional.logsigmoid(z) / tau).view(T, H, D)
    S = torch.zeros(H, D, V, dtype=F64)
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = rms_norm(out, eps, w[pre + "norm"]).reshape(T, H * V)
    g = h @ w[pre + "g"].T
    return (out * g * torch.sigmoid(g)) @ w[pre + "o"].T


def parallel_mixer(h, w, pre, p, eps):
    left = windowed_attention(h, w, pre + "left.", p["left"], eps)
    right = matrix_memory(h, w, pre + "right.", p["right"], eps)
    return p["left_scale"] * left + p["right_scale"] * right


def dense_feed_forward(h, w, pre):
    g = h @ w[pre + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


MIXERS = {"gla": gated_linear_attention, "parallel": parallel_mixer}


def owner_of(layers, i):
    """The layer whose tensors layer i uses."""
    while "weights_of" in layers[i]:
        i = layers[i]["weights_of"]
    return i


def layer_forward(x, w, cfg, i):
    entry = cfg["layers"][i]
    pre = f"l{owner_of(cfg['layers'], i)}."
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    y = MIXERS[entry["type"]](x, w, pre + "mix.", entry["mixer"], eps)
    y = y * torch.sigmoid(x @ w[pre + "rg1"].T + w[pre + "rg1.b"])
    x = rms_norm(alpha * x + y, eps, w[pre + "norm1"])
    if entry.get("mlp") is not None:
        y = dense_feed_forward(x, w, pre + "mlp.")
        y = y * torch.sigmoid(x @ w[pre + "rg2"].T + w[pre + "rg2.b"])
        x = rms_norm(alpha * x + y, eps, w[pre + "norm2"])
    return x


def forward_all(ids, w, cfg, streams=None):
    """Logits [T, vocab] of a whole sequence; `streams` (a list) receives the rows after every layer run."""
    x = w["embed"][torch.tensor(list(ids), dtype=torch.long)] * cfg["embedding"]["scale"]
    for i in range(len(cfg["layers"])):
        x = layer_forward(x, w, cfg, i)
        if streams is not None:
            streams.append(x)
    x = rms_norm(x, cfg["norm"]["eps"], w["final.norm"])
    return x @ w["head"].T


def greedy_generate(prompt, n_new, w, cfg):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward_all(ids, w, cfg)[-1])))
    return ids[len(prompt):]
