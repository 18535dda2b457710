"""Small Pasovik models for the tests: configurations that differ from each other in every size and option, and random
weights for them, written as a model folder (config.json, model.safetensors in bfloat16)."""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def attention(heads, kv_heads, dim, vdim, rot_dims, base=10000.0, factor=None, softcap=None, scale=None):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "rot": rot, "scale": scale if scale is not None else dim ** -0.5, "vdim": vdim}
    if softcap is not None:
        m["softcap"] = softcap
    return m


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, factor=None, scale=None, kv_from=None):
    rot = {"base": base, "dims": rot_dim}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot, "rot_dim": rot_dim,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def lightning(heads, dim, vdim, decay):
    assert len(decay) == heads
    return {"decay": list(decay), "dim": dim, "heads": heads, "vdim": vdim}


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def moe(experts, top, ff, limit=2.0):
    return {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "top": top}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=64, vocab=97, eps=1e-5, side=None):
    c = {"architecture": "Pasovik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if side:
        c["token_side"] = {"dim": side}
    return c


# Layers that differ from each other: grouped and ungrouped heads, key and value sizes that differ and are no multiples of
# 16, a rotation of part of a head and of all of it, with and without a stretch and a cap, two latents of different sizes
# with a reader each, linear attention with one head and with several, dense and routed feed-forwards, a layer without one,
# one expert of one, all experts chosen, a side input whose width is no whole vector.
MIXED = config([
    layer("lightning", lightning(3, 12, 20, [0.5, 0.93, 0.999]), dense(24)),
    layer("attention", attention(4, 2, 24, 40, rot_dims=8, factor=2.0, softcap=15.0), moe(3, 3, 40, limit=3.0)),
    layer("latent_attention", latent(3, 12, 6, 20, kv_rank=20, q_rank=12, base=500.0), dense(40)),
    layer("attention", attention(4, 1, 16, 16, rot_dims=16, base=77.0), None),
    layer("latent_attention", latent(2, 8, 6, 16, kv_rank=20, q_rank=10, base=500.0, scale=0.4, kv_from=2), moe(1, 1, 16, limit=0.5)),
    layer("lightning", lightning(1, 40, 8, [0.97]), dense(72)),
    # The two routers that choose stand last: where two experts all but tie, the 16-bit engine may choose the other one, and
    # a token that went to another expert in an early layer would change the keys that every later token reads.
    layer("latent_attention", latent(4, 16, 16, 8, kv_rank=48, q_rank=24, factor=8.0), moe(6, 3, 24, limit=1.5)),
    layer("latent_attention", latent(1, 24, 16, 24, kv_rank=48, q_rank=8, factor=8.0, kv_from=6), moe(5, 2, 24, limit=1.0)),
], width=64, vocab=97, side=5)
# The head size of the kernels' widest tiles, a cache row of a latent as wide, and a state as wide as a wave; no side input.
WIDE = config([layer("attention", attention(4, 2, 128, 128, rot_dims=32, base=400000.0, softcap=30.0), moe(12, 5, 64, limit=1.25)),
               layer("lightning", lightning(2, 64, 64, [0.9, 0.99]), dense(120)),
               layer("latent_attention", latent(4, 32, 16, 32, kv_rank=112, q_rank=48, base=400000.0), dense(64))], width=96, vocab=130)
CONFIGS = {"MIXED": MIXED, "WIDE": WIDE}


def random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(*shape, generator=g) * std

    def uniform(*shape, lo=-1.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    W, L = cfg["width"], len(cfg["layers"])
    w = {"embed": normal(cfg["vocab"], W), "final.norm": uniform(W, lo=0.5, hi=1.5), "head": normal(cfg["vocab"], W, std=2.0 * W ** -0.5)}
    side = cfg.get("token_side", {}).get("dim", 0)
    if side:
        w["side.embed"] = normal(cfg["vocab"], L * side)
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = spec["mixer"]
        w[p + "norm1"] = uniform(W, lo=0.2, hi=0.8)
        w[p + "norm2"] = uniform(W, lo=0.2, hi=0.8)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        if spec["type"] == "attention":
            G = m["kv_heads"]
            w[p + "mix.q"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.k"] = normal(G * d, W, std=W ** -0.5)
            w[p + "mix.v"] = normal(G * dv, W, std=W ** -0.5)
            w[p + "mix.q.norm"] = uniform(d, lo=0.5, hi=2.0)
            w[p + "mix.k.norm"] = uniform(d, lo=0.5, hi=2.0)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        elif spec["type"] == "latent_attention":
            dr, r, rq = m["rot_dim"], m["kv_rank"], m["q_rank"]
            w[p + "mix.dq"] = normal(rq, W, std=W ** -0.5)
            w[p + "mix.dq.norm"] = uniform(rq, lo=0.5, hi=2.0)
            w[p + "mix.uq"] = normal(H * (d + dr), rq, std=rq ** -0.5)
            if m.get("kv_from") is None:
                w[p + "mix.dkv"] = normal(r + dr, W, std=W ** -0.5)
                w[p + "mix.dkv.norm"] = uniform(r, lo=0.5, hi=2.0)
            w[p + "mix.uk"] = normal(H * d, r, std=r ** -0.5)
            w[p + "mix.uv"] = normal(H * dv, r, std=r ** -0.5)
            w[p + "mix.g"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        else:
            w[p + "mix.q"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.k"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.v"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.g"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
            w[p + "mix.norm"] = uniform(H * dv, lo=0.5, hi=1.5)
        mlp = spec["mlp"]
        if mlp and mlp["kind"] == "dense":
            w[p + "mlp.gate"] = normal(mlp["ff"], W, std=W ** -0.5)
            w[p + "mlp.up"] = normal(mlp["ff"], W, std=W ** -0.5)
            w[p + "mlp.down"] = normal(W, mlp["ff"], std=mlp["ff"] ** -0.5)
        elif mlp:
            E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
            w[p + "mlp.router"] = normal(E, W, std=2.0 * W ** -0.5)
            for e in range(E):
                w[p + f"mlp.e{e}.gate"] = normal(F, W, std=W ** -0.5)
                w[p + f"mlp.e{e}.up"] = normal(F, W, std=W ** -0.5)
                w[p + f"mlp.e{e}.down"] = normal(W, F, std=F ** -0.5)
        else:
            del w[p + "norm2"]
        if side:
            w[p + "side.gate"] = normal(side, W, std=W ** -0.5)
            w[p + "side.proj"] = normal(W, side, std=side ** -0.5)
            w[p + "side.norm"] = uniform(W, lo=0.1, hi=0.5)
    # What the file stores is what both sides compute with.
    return {n: t.to(torch.bfloat16).contiguous() for n, t in w.items()}


def write_model(folder, cfg, weights):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(weights, str(folder / "model.safetensors"))
    return folder
