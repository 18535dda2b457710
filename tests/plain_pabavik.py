"""A plain, slow implementation of the Pabavik design: torch on the CPU in float64, one function per mechanism, token by
token where the design is recurrent and every key where it attends.  It shares nothing with the engine.

The design: x = embed[token] * scale is the residual stream.  A layer is
    x <- x + norm_b(mixer(norm_a(x)));  x <- x + norm_d(ff(norm_c(x)))
with norms y = x / sqrt(mean(x^2) + eps) * (1 + w).  The mixer is softmax attention (grouped heads, q and k normed per
head and partly rotated, a window, one extra term exp(0) in the denominator, an output gate) or gated linear attention (a
decayed outer-product state per head).  The feed-forward is a mixture of gated experts beside a shared expert.  Then the
model's norm, the vocabulary projection, and c * tanh(logits / c).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    return rms(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return rms(x, eps) * w.to(F64)


def rotate(x, positions, dims, base):
    """x [T, heads, d]: element i of the first `dims` is paired with i + dims/2 and turned by position * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(F64)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def attention_keys(m, w, p, h, positions, eps):
    """The keys as the cache holds them (normed, rotated) and the values of a layer with projections of its own."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[p + "k"].to(F64).T).view(T, G, d)
    v = (h @ w[p + "v"].to(F64).T).view(T, G, dv)
    k = norm_plain(k, w[p + "k.norm"], eps)
    k = rotate(k, positions, m["rot"]["dims"], m["rot"]["base"])
    return k, v


def attention(m, w, p, h, eps, keys=None):
    """h [T, width] of one sequence from position 0.  keys: (k, v) of the layer named by kv_from.  Returns (out, (k, v))."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T)
    q = (h @ w[p + "q"].to(F64).T).view(T, H, d)
    q = norm_plain(q, w[p + "q.norm"], eps)
    q = rotate(q, positions, m["rot"]["dims"], m["rot"]["base"])
    k, v = keys if keys is not None else attention_keys(m, w, p, h, positions, eps)
    size = m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            lo = max(0, i - size + 1)
            s = (k[lo:i + 1, g] @ q[i, head]) * m["scale"]
            e = torch.exp(s)
            out[i, head] = (e / (1.0 + e.sum())) @ v[lo:i + 1, g]
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return (out.reshape(T, H * dv) * gate) @ w[p + "o"].to(F64).T, (k, v)


def gla(m, w, p, h, eps, state=None):
    """Gated linear attention, token by token.  state [heads, dim, vdim] or None; returns (out, state)."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].to(F64).T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].to(F64).T).view(T, H, d)
    v = (h @ w[p + "v"].to(F64).T).view(T, H, dv)
    z = (h @ w[p + "a1"].to(F64).T) @ w[p + "a2"].to(F64).T + w[p + "a2.b"].to(F64)
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = norm_plain(o, w[p + "norm"], eps)
    gate = h @ w[p + "g"].to(F64).T
    return (o.reshape(T, H * dv) * (gate * torch.sigmoid(gate))) @ w[p + "o"].to(F64).T, S


def expert(w, p, h, limit):
    g = torch.clamp(h @ w[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ w[p + "up"].to(F64).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].to(F64).T


def route(mlp, w, p, h):
    """The chosen experts [T, top] (largest logit first, the lower index on a tie) and their weights."""
    z = h @ w[p + "router"].to(F64).T + w[p + "router.b"].to(F64)
    top = mlp["router"]["top"]
    order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), dim=-1)


def experts(mlp, w, p, h):
    idx, wts = route(mlp, w, p, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            out[t] += wts[t, j] * expert(w, f"{p}e{int(idx[t, j])}.", h[t:t + 1], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + expert(w, p + "shared.", h, mlp["shared"]["limit"])
    return out


def forward(cfg, w, tokens, streams=None):
    """Logits [T, vocab] in float64 for one sequence from position 0.  streams: a list that receives the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"].to(F64)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = norm_around_zero(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            y, kept[i] = attention(m, w, p + "mix.", h, eps, kept[m["kv_from"]] if m.get("kv_from") is not None else None)
            if m.get("kv_from") is not None:
                kept[i] = kept[m["kv_from"]]
        elif layer["type"] == "gla":
            y, _ = gla(m, w, p + "mix.", h, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_around_zero(y, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = norm_around_zero(x, w[p + "norm2"], eps)
            x = x + norm_around_zero(experts(layer["mlp"], w, p + "mlp.", h), w[p + "norm2b"], eps)
        if streams is not None:
            streams.append(x.clone())
    x = norm_around_zero(x, w["final.norm"], eps)
    logits = x @ w["head"].to(F64).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def generate_greedy(cfg, w, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(torch.argmax(forward(cfg, w, seq)[-1])))
    return seq[len(prompt):]
