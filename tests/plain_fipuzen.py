"""The Fipuzen decoder written out plainly: float64, whole sequences, one function per mechanism.

Nothing here is shared with the engine: no cache, no pages, no state slots, no kernels. A sequence goes in as a list of
token ids, logits for every position come out. Tests compare the engine with this.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def w64(tensors, name):
    return tensors[name].to(F64)


def layer_norm(x, gain, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * gain + bias


def rms_norm(x, gain, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def query_temperature(T, coef, every):
    """The factor on the query at positions 0..T-1: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(T, dtype=torch.int64)
    return 1.0 + coef * torch.log(torch.div(p + 1, every, rounding_mode="floor").to(F64) + 1.0)


def sink_softmax(scores, visible):
    """Softmax over the visible keys with one more, valueless key of score 0 in the denominator."""
    s = scores.masked_fill(~visible, -math.inf)
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def plain_softmax(scores, visible):
    return torch.softmax(scores.masked_fill(~visible, -math.inf), dim=-1)


def causal(T):
    return torch.ones(T, T, dtype=torch.bool).tril()


def sink_attention(h, t, pre, m):
    """Grouped-query attention with biased projections, a position-dependent query factor, a sink in the softmax and
    a sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w64(t, pre + "q").T + w64(t, pre + "q.b")).view(T, H, D)
    k = (h @ w64(t, pre + "k").T + w64(t, pre + "k.b")).view(T, G, D)
    v = (h @ w64(t, pre + "v").T + w64(t, pre + "v.b")).view(T, G, V)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"]).view(T, 1, 1)
    gate = torch.sigmoid(h @ w64(t, pre + "g").T)                   # [T, H]
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        s = q[:, head] @ k[:, g].T * m["scale"]
        out[:, head] = sink_softmax(s, causal(T)) @ v[:, g] * gate[:, head:head + 1]
    return out.reshape(T, H * V) @ w64(t, pre + "o").T


def lightning(h, t, pre, m, eps):
    """Linear attention with a fixed decay per head, token by token from an empty state."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w64(t, pre + "q").T).view(T, H, D)
    k = silu(h @ w64(t, pre + "k").T).view(T, H, D)
    v = silu(h @ w64(t, pre + "v").T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for i in range(T):
            S = m["decay"][head] * S + torch.outer(k[i, head], v[i, head])
            o[i, head] = S.T @ q[i, head]
    y = rms_norm(o.reshape(T, H * V), w64(t, pre + "norm"), eps) * torch.sigmoid(h @ w64(t, pre + "g").T)
    return y @ w64(t, pre + "o").T


def rotate_pairs(x, positions, dims, base):
    """Turns the pairs (2i, 2i+1), i < dims/2, of the last axis by position * base^(-2i/dims); the rest stays."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F64)
    ang = positions.to(F64).view(-1, *([1] * (x.dim() - 2)), 1) * base ** (-2.0 * i / dims)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * torch.cos(ang) - b * torch.sin(ang)
    out[..., 1:dims:2] = b * torch.cos(ang) + a * torch.sin(ang)
    return out


def latent_attention(h, t, pre, m, eps):
    """Attention whose keys and values are made from a normed low-rank latent, with one rotated key part shared by
    the heads. Written the long way: keys and values of every head are built from the latent."""
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ w64(t, pre + "q").T).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    down = h @ w64(t, pre + "dkv").T
    c = rms_norm(down[:, :C], w64(t, pre + "dkv.norm"), eps)
    k_rot = rotate_pairs(down[:, C:], pos, m["rot"]["dims"], m["rot"]["base"])          # [T, R]
    k_plain = (c @ w64(t, pre + "uk").T).view(T, H, D)
    v = (c @ w64(t, pre + "uv").T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        out[:, head] = plain_softmax(s, causal(T)) @ v[:, head]
    return out.reshape(T, H * V) @ w64(t, pre + "o").T


def routed_experts(h, t, pre, mlp, margins=None):
    """Mixture of experts with identity experts at the end of the router's outputs. margins (a list) receives, per
    row, how clear the closest choice was: the gap between the last chosen and the first unchosen score over the larger
    of the two softmax values (about the change of a router output that would turn the choice)."""
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    z = h @ w64(t, pre + "router").T                                 # [T, E + I]
    s = torch.softmax(z, dim=-1)
    choice = s + w64(t, pre + "correction")
    chosen = torch.topk(choice, top, dim=-1).indices
    if margins is not None and top < E + I:
        order = torch.sort(choice, dim=-1, descending=True)
        gap = order.values[:, top - 1] - order.values[:, top]
        big = torch.maximum(torch.gather(s, 1, order.indices[:, top - 1:top]), torch.gather(s, 1, order.indices[:, top:top + 1]))
        margins.extend((gap / big[:, 0]).tolist())
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e in chosen[i].tolist():
            weight = s[i, e] * r["scale"]
            if e >= E:
                out[i] += weight * h[i]
            else:
                out[i] += weight * (w64(t, f"{pre}e{e}.down") @ gelu_erf(w64(t, f"{pre}e{e}.up") @ h[i]))
    return out


def token_side(x, tokens, t, pre, layer, dim, eps):
    """What a layer adds from its slice of the per-token side table."""
    e = w64(t, "side.embed")[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w64(t, pre + "gate").T) * e) @ w64(t, pre + "proj").T
    return rms_norm(y, w64(t, pre + "norm"), eps)


def forward(cfg, t, tokens, layer_outputs=None, margins=None):
    """Logits [T, vocab] in float64 for one sequence. cfg: the raw dictionary of config.json; t: tensors by name."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    x = w64(t, "embed")[tokens]
    side = cfg.get("token_side")
    for i, entry in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", entry["mixer"]
        h = layer_norm(x, w64(t, pre + "norm1"), w64(t, pre + "norm1.b"), eps)
        if entry["type"] == "attention":
            x = x + sink_attention(h, t, pre + "mix.", m)
        elif entry["type"] == "lightning":
            x = x + lightning(h, t, pre + "mix.", m, eps)
        elif entry["type"] == "latent_attention":
            x = x + latent_attention(h, t, pre + "mix.", m, eps)
        else:
            raise ValueError(entry["type"])
        if entry.get("mlp") is not None:
            h = layer_norm(x, w64(t, pre + "norm2"), w64(t, pre + "norm2.b"), eps)
            x = x + routed_experts(h, t, pre + "mlp.", entry["mlp"], margins)
        if side:
            x = x + token_side(x, tokens, t, pre + "side.", i, side["dim"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    x = layer_norm(x, w64(t, "final.norm"), w64(t, "final.norm.b"), eps)
    return x @ w64(t, "head").T


def greedy_generate(cfg, t, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, t, ids)[-1])))
    return ids[len(prompt):]
