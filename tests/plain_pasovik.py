"""A plain, slow implementation of the Pasovik design: torch on the CPU in float64, one function per mechanism, token by
token where the design is recurrent and every key where it attends.  It shares nothing with the engine.

The design: x = embed[token] is the residual stream.  The sublayers read the stream as it is and only their outputs are
normed:
    x <- x + n1(mixer(x));  x <- x + n2(ff(x))  (a layer may have no feed-forward);  x <- x + side(x, token)
with n(y) = y / sqrt(mean(y^2) + eps) * w.  The mixer is softmax attention (grouped heads, q and k normed per head, pairs
of neighbouring entries rotated, capped scores), attention through a latent (queries and keys/values projected down and up
again, one rotated key part for all heads, an output gate, optionally on the latent of an earlier layer) or linear attention
with a fixed decay per head.  The feed-forward is dense (silu-gated) or a mixture of clamped gated experts whose router
scores are logistic and scale the expert's input.  Then the model's norm and the vocabulary projection.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w.to(F64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(rot):
    """f_i = base^(-2i/dims), all divided by the linear scaling factor where the configuration has one."""
    dims = rot["dims"]
    f = rot["base"] ** (-2.0 * torch.arange(dims // 2, dtype=F64) / dims)
    if rot.get("scaling"):
        f = f / rot["scaling"]["factor"]
    return f


def rotate_pairs(x, positions, rot):
    """x [T, heads, d]: entries 2i and 2i + 1 of the first rot.dims form a pair that turns by position * f_i."""
    dims = rot["dims"]
    ang = positions.to(F64)[:, None] * frequencies(rot)[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def attention(m, w, p, h, eps):
    """Softmax attention of one sequence from position 0; h [T, width]."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T)
    q = (h @ w[p + "q"].to(F64).T).view(T, H, d)
    k = (h @ w[p + "k"].to(F64).T).view(T, G, d)
    v = (h @ w[p + "v"].to(F64).T).view(T, G, dv)
    q, k = norm(q, w[p + "q.norm"], eps), norm(k, w[p + "k.norm"], eps)
    if m.get("rot"):
        q, k = rotate_pairs(q, positions, m["rot"]), rotate_pairs(k, positions, m["rot"])
    out = torch.zeros(T, H, dv, dtype=F64)
    cap = m.get("softcap")
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            s = (k[:i + 1, g] @ q[i, head]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, head] = torch.softmax(s, dim=0) @ v[:i + 1, g]
    return out.reshape(T, H * dv) @ w[p + "o"].to(F64).T


def latent_keys(m, w, p, h, eps):
    """What a latent attention layer keeps of every token: the normed latent and the rotated key part."""
    T, r = h.shape[0], m["kv_rank"]
    down = h @ w[p + "dkv"].to(F64).T
    c = norm(down[:, :r], w[p + "dkv.norm"], eps)
    shared = rotate_pairs(down[:, None, r:], torch.arange(T), m["rot"])[:, 0]
    return c, shared


def latent_attention(m, w, p, h, eps, kept=None):
    """Attention through a latent; kept: (latent, rotated key part) of the layer that kv_from names.  Returns (out, kept)."""
    T = h.shape[0]
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = norm(h @ w[p + "dq"].to(F64).T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].to(F64).T).view(T, H, d + dr)
    q_flat, q_rot = q[..., :d], rotate_pairs(q[..., d:], torch.arange(T), m["rot"])
    c, shared = kept if kept is not None else latent_keys(m, w, p, h, eps)
    k = (c @ w[p + "uk"].to(F64).T).view(T, H, d)
    v = (c @ w[p + "uv"].to(F64).T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for head in range(H):
        for i in range(T):
            s = (k[:i + 1, head] @ q_flat[i, head] + shared[:i + 1] @ q_rot[i, head]) * m["scale"]
            out[i, head] = torch.softmax(s, dim=0) @ v[:i + 1, head]
    gate = torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return (out.reshape(T, H * dv) * gate) @ w[p + "o"].to(F64).T, (c, shared)


def lightning(m, w, p, h, eps, state=None):
    """Linear attention with a fixed decay per head, token by token.  state [heads, dim, vdim] or None; returns (out, state)."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].to(F64).T).view(T, H, d)
    k = silu(h @ w[p + "k"].to(F64).T).view(T, H, d)
    v = silu(h @ w[p + "v"].to(F64).T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(H, d, dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    y = norm(o.reshape(T, H * dv), w[p + "norm"], eps) * torch.sigmoid(h @ w[p + "g"].to(F64).T)
    return y @ w[p + "o"].to(F64).T, S


def dense(w, p, h):
    return (silu(h @ w[p + "gate"].to(F64).T) * (h @ w[p + "up"].to(F64).T)) @ w[p + "down"].to(F64).T


def expert(w, p, h, limit):
    g = torch.clamp(h @ w[p + "gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ w[p + "up"].to(F64).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].to(F64).T


def route(mlp, w, p, h):
    """The chosen experts [T, top] (largest score first, the lower index on a tie) and their logistic scores."""
    s = torch.sigmoid(h @ w[p + "router"].to(F64).T)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :mlp["router"]["top"]]
    return order, torch.gather(s, 1, order)


def experts(mlp, w, p, h):
    """sum over the chosen of expert(score * h): the score scales what the expert reads."""
    idx, wts = route(mlp, w, p, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            out[t] += expert(w, f"{p}e{int(idx[t, j])}.", wts[t, j] * h[t:t + 1], mlp["expert"]["limit"])[0]
    return out


def token_side(cfg, w, i, x, tokens, eps):
    """What layer i adds from the token's own second embedding: its slice of the table, gated by the stream."""
    n = cfg["token_side"]["dim"]
    e = w["side.embed"].to(F64)[torch.tensor(tokens), i * n:(i + 1) * n]
    g = gelu_tanh(x @ w[f"l{i}.side.gate"].to(F64).T) * e
    return norm(g @ w[f"l{i}.side.proj"].to(F64).T, w[f"l{i}.side.norm"], eps)


def forward(cfg, w, tokens, streams=None):
    """Logits [T, vocab] in float64 for one sequence from position 0.  streams: a list that receives the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"].to(F64)[torch.tensor(tokens)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        if layer["type"] == "attention":
            y = attention(m, w, p + "mix.", x, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            y, kept[i] = latent_attention(m, w, p + "mix.", x, eps, kept[src] if src is not None else None)
        elif layer["type"] == "lightning":
            y, _ = lightning(m, w, p + "mix.", x, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm(y, w[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp:
            y = dense(w, p + "mlp.", x) if mlp["kind"] == "dense" else experts(mlp, w, p + "mlp.", x)
            x = x + norm(y, w[p + "norm2"], eps)
        if cfg.get("token_side"):
            x = x + token_side(cfg, w, i, x, tokens, eps)
        if streams is not None:
            streams.append(x.clone())
    return norm(x, w["final.norm"], eps) @ w["head"].to(F64).T


def generate_greedy(cfg, w, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(torch.argmax(forward(cfg, w, seq)[-1])))
    return seq[len(prompt):]
