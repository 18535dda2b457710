"""The Pabavik architecture on the CPU: what the native library makes of its config.json, and the plain implementation's
own pieces against torch's routines and equations written out."""
import json
import math
import subprocess

import pytest
import torch

import plain_pabavik as plain
from pabavik_models import MIXED, attention, config, gla, layer, moe, random_weights, write_model
from vosti_amd.config import ConfigError, config_from_dict
from vosti_amd.kernels import build

F64 = torch.float64


def test_description_of_a_configuration():
    c = config_from_dict(MIXED)
    assert c.architecture == "Pabavik" and c.vocab == 97 and c.width == 64 and c.layers == 6 and c.embedding_scale == 4.0 and c.logit_softcap == 20.0
    spec = c.model_spec()
    assert [l.block for l in spec.layers] == ["sandwich"] * 6
    assert [l.mixer.kind for l in spec.layers] == ["gated_linear_attention", "attention", "attention", "attention", "gated_linear_attention", "attention"]
    assert [l.feed_forward.kind for l in spec.layers] == ["routed_experts", "routed_experts", "none", "routed_experts", "routed_experts", "routed_experts"]
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(0, None), (1, None), (2, 1), (3, None), (4, None), (5, 3)]
    assert spec.embedding.kind == "token_embedding_scaled" and spec.embedding.params["scale"] == 4.0
    assert spec.final_norm.params == {"size": 64, "eps": 1e-5, "offset": 1}
    assert spec.head.params["softcap"] == 20.0
    assert spec.names["head.weight"] == "head" and spec.names["embedding.weight"] == "embed"
    f = spec.layers[0].feed_forward.params
    assert (f["experts"], f["top"], f["intermediate_size"], f["limit"], f["shared_size"], f["shared_limit"], f["router_bias"], f["gated"]) == (5, 2, 24, 1.0, 40, 0.7, 1, 1)
    assert (f["glu_slope"], f["up_shift"]) == (1.702, 1)
    assert "shared_size" not in spec.layers[1].feed_forward.params
    n = spec.layers[0].names
    assert n["feed_forward.experts.4.gate_proj.weight"] == "l0.mlp.e4.gate" and n["feed_forward.shared.down_proj.weight"] == "l0.mlp.shared.down"
    assert n["feed_forward.router.bias"] == "l0.mlp.router.b" and n["mixer.decay_up.bias"] == "l0.mix.a2.b" and n["mixer.out_norm.weight"] == "l0.mix.norm"
    assert n["norms.mixer_out.weight"] == "l0.norm1b" and n["norms.ffn_out.weight"] == "l0.norm2b"
    assert "norms.ffn_in.weight" not in spec.layers[2].names


def test_the_mixers_in_the_library_s_own_words():
    from vosti_amd.config.registry import describe
    d = describe(MIXED)
    a = d["layers"][1]["mixer"]
    n = a["numbers"]
    assert (n["num_heads"], n["num_kv_heads"], n["head_dim"], n["value_dim"], n["window"], n["sink"], n["exact_weights"], n["output_gate"], n["own_kv"]) == \
        (4, 2, 24, 40, 19, 2, 1, 1, 1)
    assert a["parts"]["q_norm"]["numbers"] == {"size": 24, "eps": 1e-5} and a["parts"]["k_norm"]["kind"] == "rmsnorm"
    r = a["parts"]["position"]
    assert r["kind"] == "rotary_stretched" and (r["numbers"]["rotary_dim"], r["numbers"]["theta"]) == (8, 10000) and "factor" not in r["numbers"]
    b = d["layers"][2]["mixer"]
    assert b["numbers"]["own_kv"] == 0 and b["numbers"]["window"] == 33 and b["numbers"]["scale"] == 0.3 and "k_norm" not in b["parts"]
    assert "mixer.k_proj.weight" not in d["layers"][2]["names"] and d["layers"][2]["names"]["mixer.gate_proj.weight"] == "l2.mix.g"
    g = d["layers"][4]["mixer"]["numbers"]
    assert (g["num_heads"], g["key_dim"], g["value_dim"], g["decay_root"]) == (1, 40, 8, 16)


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][1].update(type="serial"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "keys of its own"),
    (lambda c: c["layers"][5]["mixer"].update(kv_from=2), "keys of its own"),
    (lambda c: c["layers"][2]["mixer"].update(dim=32), "differs"),
    (lambda c: c["layers"][0]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "moe"),
    (lambda c: c.pop("embedding"), "embedding"),
])
def test_configuration_errors_name_the_key(change, text):
    cfg = json.loads(json.dumps(MIXED))
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


def test_tensor_names_are_the_files(tmp_path):
    """The program's own description of a model folder lists exactly the tensors that such a file holds (a layer without
    a feed-forward has no use for its second pair of norms; a file may hold them all the same)."""
    w = random_weights(MIXED, 1)
    folder = write_model(tmp_path / "m", MIXED, w)
    program = str(build.ensure("engine", verbose=False))
    r = subprocess.run([program, "--kind", "describe", "--model-path", str(folder)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert got["architecture"] == "Pabavik"
    assert got["tensor_names"] == sorted(n for n in w if n not in ("l2.norm2", "l2.norm2b"))


# ------------------------------------------------------------------------- the plain implementation's own pieces
def test_norms_against_torch():
    x = torch.randn(5, 12, dtype=F64, generator=torch.Generator().manual_seed(0))
    w = torch.randn(12, dtype=F64, generator=torch.Generator().manual_seed(1)) * 0.1
    ref = torch.nn.functional.rms_norm(x, (12,), eps=1e-5)
    assert torch.allclose(plain.norm_around_zero(x, w, 1e-5), ref * (1 + w), atol=1e-12)
    assert torch.allclose(plain.norm_plain(x, w, 1e-5), ref * w, atol=1e-12)


def test_rotation_keeps_what_it_does_not_turn_and_turns_pairs_half_apart():
    x = torch.randn(5, 2, 12, dtype=F64, generator=torch.Generator().manual_seed(0))
    y = plain.rotate(x, torch.arange(5), 4, 100.0)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    a = 3 * 100.0 ** (-2 * 1 / 4)                                # position 3, pair 1: elements 1 and 3
    assert torch.allclose(y[3, :, 1], x[3, :, 1] * math.cos(a) - x[3, :, 3] * math.sin(a))
    assert torch.allclose(y[3, :, 3], x[3, :, 3] * math.cos(a) + x[3, :, 1] * math.sin(a))
    # A rotation of both by the same angle leaves a dot product alone: scores depend on the distance only.
    q, k = x[:1].expand(5, 2, 12), x[1:2].expand(5, 2, 12)
    d = (plain.rotate(q, torch.arange(5) + 7, 4, 100.0) * plain.rotate(k, torch.arange(5) + 4, 4, 100.0)).sum(-1)
    assert torch.allclose(d, d[:1].expand_as(d))


def one_layer(kind, mixer, mlp=None, width=8):
    cfg = config([layer(kind, mixer, mlp)], width=width, vocab=10)
    return cfg, {n: t.double() for n, t in random_weights(cfg, 2, rank=3).items()}


def test_attention_written_out():
    """One head, three tokens, a window of two: p = exp(s) / (1 + sum over the window of exp(s)), then the gate."""
    cfg, w = one_layer("attention", attention(1, 1, 4, 6, size=2, rot_dims=2, scale=0.5))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(3, 8, dtype=F64, generator=torch.Generator().manual_seed(1))
    got, (keys, values) = plain.attention(m, w, p, h, 1e-5)
    pos = torch.arange(3)
    q = plain.rotate(plain.norm_plain((h @ w[p + "q"].T).view(3, 1, 4), w[p + "q.norm"], 1e-5), pos, 2, 10000.0)[:, 0]
    k = plain.rotate(plain.norm_plain((h @ w[p + "k"].T).view(3, 1, 4), w[p + "k.norm"], 1e-5), pos, 2, 10000.0)[:, 0]
    v = h @ w[p + "v"].T
    assert torch.allclose(keys[:, 0], k) and torch.allclose(values[:, 0], v)
    e = lambda i, j: math.exp(float(q[i] @ k[j]) * 0.5)
    rows = [e(0, 0) / (1 + e(0, 0)) * v[0], (e(1, 0) * v[0] + e(1, 1) * v[1]) / (1 + e(1, 0) + e(1, 1)),
            (e(2, 1) * v[1] + e(2, 2) * v[2]) / (1 + e(2, 1) + e(2, 2))]            # the third token no longer sees the first
    want = (torch.stack(rows) * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert torch.allclose(got, want, atol=1e-12)


def test_a_layer_on_the_keys_of_another_uses_them_as_they_are():
    cfg, w = one_layer("attention", attention(2, 1, 4, 4, size=3, rot_dims=4))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(6, 8, dtype=F64, generator=torch.Generator().manual_seed(2))
    own, kept = plain.attention(m, w, p, h, 1e-5)
    other = torch.randn(6, 8, dtype=F64, generator=torch.Generator().manual_seed(3))
    again, _ = plain.attention(m, w, p, h, 1e-5, keys=plain.attention(m, w, p, other, 1e-5)[1])
    assert not torch.allclose(own, again)
    assert torch.allclose(plain.attention(m, w, p, h, 1e-5, keys=kept)[0], own)


def test_linear_attention_as_a_sum_over_the_past():
    """o_t = sum over s <= t of (q_t . (alpha_(s+1) * ... * alpha_t * k_s)) v_s per head, alpha = sigmoid(z)^(1 / tau)."""
    cfg, w = one_layer("gla", gla(2, 3, 4, tau=5.0))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(6, 8, dtype=F64, generator=torch.Generator().manual_seed(1))
    got, state = plain.gla(m, w, p, h, 1e-5)
    q, k, v = (h @ w[p + "q"].T).view(6, 2, 3) * 3 ** -0.5, (h @ w[p + "k"].T).view(6, 2, 3), (h @ w[p + "v"].T).view(6, 2, 4)
    alpha = torch.sigmoid((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]).view(6, 2, 3) ** (1 / 5.0)
    o = torch.zeros(6, 2, 4, dtype=F64)
    for t in range(6):
        for s in range(t + 1):
            decay = alpha[s + 1:t + 1].prod(0)
            o[t] += ((q[t] * decay * k[s]).sum(-1))[:, None] * v[s]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * w[p + "norm"]
    gate = h @ w[p + "g"].T
    assert torch.allclose(got, (o.reshape(6, 8) * torch.nn.functional.silu(gate)) @ w[p + "o"].T, atol=1e-10)
    # The state that is carried: two halves of a sequence give what the whole gives.
    first, s1 = plain.gla(m, w, p, h[:2], 1e-5)
    second, s2 = plain.gla(m, w, p, h[2:], 1e-5, state=s1)
    assert torch.allclose(torch.cat([first, second]), got, atol=1e-12) and torch.allclose(s2, state, atol=1e-12)


def test_routing_is_a_softmax_over_the_chosen_logits():
    cfg, w = one_layer("gla", gla(1, 2, 2), moe(5, 2, 6))
    mlp, p = cfg["layers"][0]["mlp"], "l0.mlp."
    h = torch.randn(9, 8, dtype=F64, generator=torch.Generator().manual_seed(3))
    idx, wt = plain.route(mlp, w, p, h)
    z = h @ w[p + "router"].T + w[p + "router.b"]
    for t in range(9):
        order = sorted(range(5), key=lambda e: -float(z[t, e]))[:2]
        assert idx[t].tolist() == order
        assert torch.allclose(wt[t], torch.softmax(z[t, order], 0))
    # The bias decides: a large one on the last expert puts it first everywhere.
    w[p + "router.b"][4] = 100.0
    assert plain.route(mlp, w, p, h)[0][:, 0].tolist() == [4] * 9


def test_an_expert_written_out():
    cfg, w = one_layer("gla", gla(1, 2, 2), moe(3, 1, 5, limit=0.3, shared=(4, 0.2)))
    mlp, p = cfg["layers"][0]["mlp"], "l0.mlp."
    h = torch.randn(4, 8, dtype=F64, generator=torch.Generator().manual_seed(5)) * 3

    def one(name, x, limit):
        g, u = w[p + name + ".gate"] @ x, w[p + name + ".up"] @ x
        g, u = torch.minimum(g, torch.tensor(limit, dtype=F64)), u.clamp(-limit, limit)
        assert (g < -limit).any() or True                           # the gate is bounded above only
        return w[p + name + ".down"] @ (g / (1 + torch.exp(-1.702 * g)) * (u + 1))

    got = plain.experts(mlp, w, p, h)
    z = h @ w[p + "router"].T + w[p + "router.b"]
    for t in range(4):
        e = int(z[t].argmax())
        assert torch.allclose(got[t], one(f"e{e}", h[t], 0.3) + one("shared", h[t], 0.2), atol=1e-12)
    assert float((h @ w[p + "e0.gate"].T).min()) < -0.3                 # the test's inputs do reach below the lower limit


def test_the_cap_on_the_logits():
    cfg, w = one_layer("gla", gla(1, 2, 2))
    tokens = [1, 2, 3]
    capped = plain.forward(cfg, w, tokens)
    free = plain.forward(dict(cfg, logit_softcap=None), w, tokens)
    assert torch.allclose(capped, 20.0 * torch.tanh(free / 20.0)) and capped.abs().max() < 20.0
