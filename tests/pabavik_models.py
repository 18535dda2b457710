"""Small Pabavik models for the tests: configurations that differ from each other in every size and option, and random
weights for them, written as a model folder (config.json, model.safetensors in bfloat16)."""
from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def attention(heads, kv_heads, dim, vdim, size, rot_dims, base=10000.0, scale=None, kv_from=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "mask": {"size": size}, "rot": {"base": base, "dims": rot_dims},
         "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def gla(heads, dim, vdim, tau=8.0):
    return {"dim": dim, "heads": heads, "tau": tau, "vdim": vdim}


def moe(experts, top, ff, limit=2.0, shared=None):
    m = {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=64, vocab=97, embed_scale=4.0, eps=1e-5, softcap=20.0):
    return {"architecture": "Pabavik", "embedding": {"scale": embed_scale}, "layers": layers, "logit_softcap": softcap, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


# Layers that differ from each other: grouped and ungrouped heads, key and value sizes that differ and are no multiples of
# 16, a rotation of part of a head and of all of it, windows that end inside pages, a layer on the keys of another, linear
# attention with one head and with several, a layer without a feed-forward, experts with and without a shared one, one
# expert of one, all experts chosen.
MIXED = config([
    layer("gla", gla(3, 12, 20, tau=4.0), moe(5, 2, 24, limit=1.0, shared=(40, 0.7))),
    layer("attention", attention(4, 2, 24, 40, size=19, rot_dims=8), moe(6, 3, 24, limit=1.5)),
    layer("attention", attention(2, 2, 24, 40, size=33, rot_dims=8, scale=0.3, kv_from=1), None),
    layer("attention", attention(4, 1, 16, 16, size=7, rot_dims=4, base=77.0), moe(3, 3, 40, limit=3.0, shared=(16, 2.0))),
    layer("gla", gla(1, 40, 8, tau=16.0), moe(1, 1, 16, limit=0.5)),
    layer("attention", attention(8, 1, 16, 16, size=64, rot_dims=4, base=77.0, kv_from=3), moe(4, 1, 8, shared=(8, 1.0))),
], width=64, vocab=97)
# One layer of each kind with the head size of the kernels' widest tiles, and a state as wide as a wave.
WIDE = config([layer("attention", attention(4, 2, 128, 128, size=150, rot_dims=32, base=250000.0), moe(8, 2, 72, shared=(120, 0.9))),
               layer("gla", gla(2, 64, 64), moe(12, 5, 64, limit=1.25)),
               layer("attention", attention(4, 2, 128, 128, size=70, rot_dims=32, base=250000.0, kv_from=0), None)], width=96, vocab=130, embed_scale=9.0)
CONFIGS = {"MIXED": MIXED, "WIDE": WIDE}
RANK = 6      # of the decay's two projections; no key of the configuration holds it


def random_weights(cfg, seed, rank=RANK):
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(*shape, generator=g) * std

    def uniform(*shape, lo=-1.0, hi=1.0):
        return torch.rand(*shape, generator=g) * (hi - lo) + lo

    W = cfg["width"]
    w = {"embed": normal(cfg["vocab"], W, std=1.0 / cfg["embedding"]["scale"]), "final.norm": uniform(W, lo=-0.3, hi=0.3),
         "head": normal(cfg["vocab"], W, std=2.0 * W ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = spec["mixer"]
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            w[p + n] = uniform(W, lo=-0.3, hi=0.3)
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        if spec["type"] == "attention":
            G = m["kv_heads"]
            w[p + "mix.q"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.q.norm"] = uniform(d, lo=0.5, hi=2.0)
            if m.get("kv_from") is None:
                w[p + "mix.k"] = normal(G * d, W, std=W ** -0.5)
                w[p + "mix.k.norm"] = uniform(d, lo=0.5, hi=2.0)
                w[p + "mix.v"] = normal(G * dv, W, std=W ** -0.5)
            w[p + "mix.g"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        else:
            w[p + "mix.q"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.k"] = normal(H * d, W, std=W ** -0.5)
            w[p + "mix.v"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.g"] = normal(H * dv, W, std=W ** -0.5)
            w[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
            w[p + "mix.norm"] = uniform(dv, lo=0.5, hi=1.5)
            w[p + "mix.a1"] = normal(rank, W, std=W ** -0.5)
            w[p + "mix.a2"] = normal(H * d, rank, std=2.0 * rank ** -0.5)
            w[p + "mix.a2.b"] = uniform(H * d, lo=0.0, hi=4.0)
        if spec["mlp"]:
            E, F = spec["mlp"]["router"]["experts"], spec["mlp"]["expert"]["ff"]
            w[p + "mlp.router"] = normal(E, W, std=2.0 * W ** -0.5)
            w[p + "mlp.router.b"] = normal(E, std=0.5)
            sizes = [(f"e{e}", F) for e in range(E)] + ([("shared", spec["mlp"]["shared"]["ff"])] if spec["mlp"].get("shared") else [])
            for name, ff in sizes:
                w[p + f"mlp.{name}.gate"] = normal(ff, W, std=2.0 * W ** -0.5)
                w[p + f"mlp.{name}.up"] = normal(ff, W, std=2.0 * W ** -0.5)
                w[p + f"mlp.{name}.down"] = normal(W, ff, std=ff ** -0.5)
    # What the file stores is what both sides compute with.
    return {n: t.to(torch.bfloat16).contiguous() for n, t in w.items()}


def write_model(folder, cfg, weights):
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(weights, str(folder / "model.safetensors"))
    return folder
