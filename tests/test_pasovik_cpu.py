"""The Pasovik architecture on the CPU: what the native library makes of its config.json, and the plain implementation's
own pieces against torch's routines and equations written out."""
import json
import math
import subprocess

import numpy as np
import pytest
import torch

import plain_pasovik as plain
from pasovik_models import MIXED, attention, config, dense, latent, layer, lightning, moe, random_weights, write_model
from vosti_amd.config import ConfigError, config_from_dict
from vosti_amd.kernels import build

F64 = torch.float64


def test_description_of_a_configuration():
    c = config_from_dict(MIXED)
    assert c.architecture == "Pasovik" and c.vocab == 97 and c.width == 64 and c.layers == 8 and c.token_side == 5
    spec = c.model_spec()
    assert [l.block for l in spec.layers] == ["post_norm"] * 8
    assert [l.mixer.kind for l in spec.layers] == ["fixed_decay_attention", "attention", "latent_attention", "attention", "latent_attention",
                                                   "fixed_decay_attention", "latent_attention", "latent_attention"]
    assert [l.feed_forward.kind for l in spec.layers] == ["swiglu", "routed_experts", "swiglu", "none", "routed_experts", "swiglu", "routed_experts", "routed_experts"]
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, None), (4, 2), (5, None), (6, None), (7, 6)]
    assert spec.embedding.kind == "token_embedding_scaled" and spec.embedding.params["scale"] == 1
    assert spec.final_norm.params == {"size": 64, "eps": 1e-5}
    assert "softcap" not in spec.head.params
    f = spec.layers[7].feed_forward.params
    assert (f["experts"], f["top"], f["intermediate_size"], f["limit"], f["gated"], f["score"], f["weigh_input"]) == (5, 2, 24, 1.0, 1, 1, 1)
    assert (f["glu_slope"], f["up_shift"]) == (1.702, 1) and "router_bias" not in f and "shared_size" not in f
    n = spec.layers[7].names
    assert n["feed_forward.experts.4.gate_proj.weight"] == "l7.mlp.e4.gate" and n["feed_forward.router.weight"] == "l7.mlp.router"
    assert n["norms.mixer_out.weight"] == "l7.norm1" and n["norms.ffn_out.weight"] == "l7.norm2" and n["norms.side_out.weight"] == "l7.side.norm"
    assert n["side.table"] == "side.embed" and n["side.gate_proj.weight"] == "l7.side.gate" and n["side.out_proj.weight"] == "l7.side.proj"
    assert spec.layers[2].names["feed_forward.down_proj.weight"] == "l2.mlp.down"
    assert "norms.ffn_out.weight" not in spec.layers[3].names


def test_the_parts_in_the_library_s_own_words():
    from vosti_amd.config.registry import describe
    d = describe(MIXED)
    a = d["layers"][1]["mixer"]
    n = a["numbers"]
    assert (n["num_heads"], n["num_kv_heads"], n["head_dim"], n["value_dim"], n["softcap"], n["exact_weights"]) == (4, 2, 24, 40, 15, 1)
    assert "window" not in n and "sink" not in n and "output_gate" not in n
    assert a["parts"]["q_norm"]["numbers"] == {"size": 24, "eps": 1e-5} and a["parts"]["k_norm"]["kind"] == "rmsnorm"
    r = a["parts"]["position"]
    assert r["kind"] == "rotary_stretched" and (r["numbers"]["rotary_dim"], r["numbers"]["theta"], r["numbers"]["linear_factor"], r["numbers"]["neighbours"]) == (8, 10000, 2, 1)
    assert d["layers"][3]["mixer"]["numbers"]["softcap"] == 0 and d["layers"][3]["mixer"]["parts"]["position"]["numbers"]["linear_factor"] == 1
    m = d["layers"][2]["mixer"]["numbers"]
    assert (m["num_heads"], m["head_dim"], m["rotary_dim"], m["value_dim"], m["kv_rank"], m["q_rank"], m["own_kv"], m["output_gate"]) == (3, 12, 6, 20, 20, 12, 1, 1)
    b = d["layers"][4]
    assert b["mixer"]["numbers"]["own_kv"] == 0 and b["mixer"]["numbers"]["scale"] == 0.4
    assert "mixer.kv_down.weight" not in b["names"] and b["names"]["mixer.k_up.weight"] == "l4.mix.uk" and b["names"]["mixer.q_down_norm.weight"] == "l4.mix.dq.norm"
    g = d["layers"][0]["mixer"]["numbers"]
    assert (g["num_heads"], g["key_dim"], g["value_dim"], g["decay.0"], g["decay.2"]) == (3, 12, 20, 0.5, 0.999)
    s = d["layers"][6]["block_numbers"]
    assert (s["side_dim"], s["side_first"], s["side_width"], s["vocab_size"]) == (5, 30, 40, 97)
    plainer = json.loads(json.dumps(MIXED))
    del plainer["token_side"]
    assert "side_dim" not in describe(plainer)["layers"][0]["block_numbers"]


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][1].update(type="serial"), "unknown mixer type"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("rot"), "rot"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0), "factor"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=4), "earlier"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=1), "latent of its own"),
    (lambda c: c["layers"][7]["mixer"].update(kv_from=4), "latent of its own"),
    (lambda c: c["layers"][4]["mixer"].update(kv_rank=24), "differs"),
    (lambda c: c["layers"][4]["mixer"]["rot"].update(base=600.0), "rotation differs"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5]), "one number a head"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5, 0.5, 1.5]), "between 0 and 1"),
    (lambda c: c["layers"][6]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][6]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "dense"),
    (lambda c: c["layers"][2]["mlp"].pop("ff"), "ff"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["token_side"].update(dim=0), "dim"),
])
def test_configuration_errors_name_the_key(change, text):
    cfg = json.loads(json.dumps(MIXED))
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


def test_tensor_names_are_the_files(tmp_path):
    """The program's own description of a model folder lists exactly the tensors that such a file holds."""
    w = random_weights(MIXED, 1)
    folder = write_model(tmp_path / "m", MIXED, w)
    program = str(build.ensure("engine", verbose=False))
    r = subprocess.run([program, "--kind", "describe", "--model-path", str(folder)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    got = json.loads(r.stdout)
    assert got["architecture"] == "Pasovik"
    assert got["tensor_names"] == sorted(w)


def test_the_rotation_frequencies_are_the_plain_ones():
    from vosti_amd.cache.host import rotary_linear_frequencies
    for base, dims, factor in ((10000.0, 8, None), (400000.0, 40, 3.0), (77.0, 2, 2.5)):
        rot = {"base": base, "dims": dims}
        if factor:
            rot["scaling"] = {"factor": factor}
        got = rotary_linear_frequencies(base, dims, factor or 1.0)
        assert np.allclose(got, plain.frequencies(rot).numpy(), rtol=1e-7, atol=0)


# ------------------------------------------------------------------------- the plain implementation's own pieces
def test_norm_and_activations_against_torch():
    x = torch.randn(5, 12, dtype=F64, generator=torch.Generator().manual_seed(0))
    w = torch.randn(12, dtype=F64, generator=torch.Generator().manual_seed(1))
    assert torch.allclose(plain.norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (12,), eps=1e-5) * w, atol=1e-12)
    assert torch.allclose(plain.gelu_tanh(x), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-12)
    assert torch.allclose(plain.silu(x), torch.nn.functional.silu(x), atol=1e-12)


def test_rotation_turns_neighbours_and_keeps_the_rest():
    x = torch.randn(5, 2, 12, dtype=F64, generator=torch.Generator().manual_seed(0))
    rot = {"base": 100.0, "dims": 4, "scaling": {"factor": 2.0}}
    y = plain.rotate_pairs(x, torch.arange(5), rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    a = 3 * 100.0 ** (-2 * 1 / 4) / 2.0                          # position 3, pair 1: elements 2 and 3
    assert torch.allclose(y[3, :, 2], x[3, :, 2] * math.cos(a) - x[3, :, 3] * math.sin(a))
    assert torch.allclose(y[3, :, 3], x[3, :, 3] * math.cos(a) + x[3, :, 2] * math.sin(a))
    # A rotation of both by the same angle leaves a dot product alone: scores depend on the distance only.
    q, k = x[:1].expand(5, 2, 12), x[1:2].expand(5, 2, 12)
    d = (plain.rotate_pairs(q, torch.arange(5) + 7, rot) * plain.rotate_pairs(k, torch.arange(5) + 4, rot)).sum(-1)
    assert torch.allclose(d, d[:1].expand_as(d))


def one_layer(kind, mixer, mlp=None, width=8, side=None):
    cfg = config([layer(kind, mixer, mlp)], width=width, vocab=10, side=side)
    return cfg, {n: t.double() for n, t in random_weights(cfg, 2).items()}


def test_attention_written_out():
    """One head, three tokens: capped scores, an ordinary softmax over the keys so far."""
    cfg, w = one_layer("attention", attention(1, 1, 4, 6, rot_dims=2, scale=2.5, softcap=1.5))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(3, 8, dtype=F64, generator=torch.Generator().manual_seed(1))
    got = plain.attention(m, w, p, h, 1e-5)
    pos = torch.arange(3)
    q = plain.rotate_pairs(plain.norm((h @ w[p + "q"].T).view(3, 1, 4), w[p + "q.norm"], 1e-5), pos, m["rot"])[:, 0]
    k = plain.rotate_pairs(plain.norm((h @ w[p + "k"].T).view(3, 1, 4), w[p + "k.norm"], 1e-5), pos, m["rot"])[:, 0]
    v = h @ w[p + "v"].T
    e = lambda i, j: math.exp(1.5 * math.tanh(float(q[i] @ k[j]) * 2.5 / 1.5))
    rows = [v[0], (e(1, 0) * v[0] + e(1, 1) * v[1]) / (e(1, 0) + e(1, 1)), (e(2, 0) * v[0] + e(2, 1) * v[1] + e(2, 2) * v[2]) / (e(2, 0) + e(2, 1) + e(2, 2))]
    assert torch.allclose(got, torch.stack(rows) @ w[p + "o"].T, atol=1e-12)
    assert max(abs(float(q[i] @ k[j]) * 2.5) for i in range(3) for j in range(3)) > 1.5       # the cap does bind here


def test_latent_attention_is_attention_over_the_latent():
    """The same scores and outputs from the cached row alone: (W_uk^T q_flat) . c + q_rot . k_rot, and W_uv (sum p c)."""
    cfg, w = one_layer("latent_attention", latent(2, 4, 2, 6, kv_rank=5, q_rank=3, base=50.0, factor=2.0))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(4, 8, dtype=F64, generator=torch.Generator().manual_seed(1))
    got, (c, shared) = plain.latent_attention(m, w, p, h, 1e-5)
    assert c.shape == (4, 5) and shared.shape == (4, 2)
    q = (plain.norm(h @ w[p + "dq"].T, w[p + "dq.norm"], 1e-5) @ w[p + "uq"].T).view(4, 2, 6)
    out = torch.zeros(4, 2, 6, dtype=F64)
    for head in range(2):
        uk, uv = w[p + "uk"][head * 4:(head + 1) * 4], w[p + "uv"][head * 6:(head + 1) * 6]
        for i in range(4):
            q_rot = plain.rotate_pairs(q[i:i + 1, head:head + 1, 4:], torch.tensor([i]), m["rot"])[0, 0]
            s = (c[:i + 1] @ (uk.T @ q[i, head, :4]) + shared[:i + 1] @ q_rot) * m["scale"]
            out[i, head] = uv @ (torch.softmax(s, 0) @ c[:i + 1])
    want = (out.reshape(4, 12) * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T
    assert torch.allclose(got, want, atol=1e-12)
    # A layer on another's latent uses it as it is.
    other = torch.randn(4, 8, dtype=F64, generator=torch.Generator().manual_seed(3))
    again, _ = plain.latent_attention(m, w, p, h, 1e-5, kept=plain.latent_keys(m, w, p, other, 1e-5))
    assert not torch.allclose(again, got)
    assert torch.allclose(plain.latent_attention(m, w, p, h, 1e-5, kept=(c, shared))[0], got)


def test_linear_attention_as_a_sum_over_the_past():
    """o_t = sum over s <= t of decay^(t - s) (q_t . k_s) v_s per head; one norm over all heads."""
    cfg, w = one_layer("lightning", lightning(2, 3, 4, [0.5, 0.9]))
    m, p = cfg["layers"][0]["mixer"], "l0.mix."
    h = torch.randn(6, 8, dtype=F64, generator=torch.Generator().manual_seed(1))
    got, state = plain.lightning(m, w, p, h, 1e-5)
    silu = torch.nn.functional.silu
    q, k, v = silu(h @ w[p + "q"].T).view(6, 2, 3), silu(h @ w[p + "k"].T).view(6, 2, 3), silu(h @ w[p + "v"].T).view(6, 2, 4)
    o = torch.zeros(6, 2, 4, dtype=F64)
    for t in range(6):
        for s in range(t + 1):
            o[t] += (torch.tensor([0.5, 0.9], dtype=F64) ** (t - s) * (q[t] * k[s]).sum(-1))[:, None] * v[s]
    o = o.reshape(6, 8)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5) * w[p + "norm"]
    assert torch.allclose(got, (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T, atol=1e-10)
    first, s1 = plain.lightning(m, w, p, h[:2], 1e-5)
    second, s2 = plain.lightning(m, w, p, h[2:], 1e-5, state=s1)
    assert torch.allclose(torch.cat([first, second]), got, atol=1e-12) and torch.allclose(s2, state, atol=1e-12)


def test_routing_scores_are_logistic_and_scale_the_input():
    cfg, w = one_layer("lightning", lightning(1, 2, 2, [0.5]), moe(5, 2, 6, limit=0.3))
    mlp, p = cfg["layers"][0]["mlp"], "l0.mlp."
    h = torch.randn(9, 8, dtype=F64, generator=torch.Generator().manual_seed(3)) * 3
    idx, wt = plain.route(mlp, w, p, h)
    z = h @ w[p + "router"].T
    got = plain.experts(mlp, w, p, h)
    for t in range(9):
        order = sorted(range(5), key=lambda e: -float(z[t, e]))[:2]
        assert idx[t].tolist() == order
        assert torch.allclose(wt[t], 1 / (1 + torch.exp(-z[t, order])))
        want = torch.zeros(8, dtype=F64)
        for e, s in zip(order, wt[t]):
            x = s * h[t]
            g, u = torch.clamp(w[p + f"e{e}.gate"] @ x, max=0.3), torch.clamp(w[p + f"e{e}.up"] @ x, -0.3, 0.3)
            want += w[p + f"e{e}.down"] @ (g / (1 + torch.exp(-1.702 * g)) * (u + 1))
        assert torch.allclose(got[t], want, atol=1e-12)
    assert float((h @ w[p + "e0.gate"].T).min()) < -0.3                 # the gate is bounded above only, and the inputs reach below


def test_the_side_input_and_the_order_of_a_layer():
    cfg, w = one_layer("lightning", lightning(1, 2, 2, [0.5]), dense(6), side=3)
    tokens = [1, 2, 3, 1]
    streams = []
    logits = plain.forward(cfg, w, tokens, streams)
    x = w["embed"][torch.tensor(tokens)]
    x = x + plain.norm(plain.lightning(cfg["layers"][0]["mixer"], w, "l0.mix.", x, 1e-5)[0], w["l0.norm1"], 1e-5)
    x = x + plain.norm(plain.dense(w, "l0.mlp.", x), w["l0.norm2"], 1e-5)
    e = w["side.embed"][torch.tensor(tokens)]
    y = (torch.nn.functional.gelu(x @ w["l0.side.gate"].T, approximate="tanh") * e) @ w["l0.side.proj"].T
    x = x + y / torch.sqrt((y * y).mean(-1, keepdim=True) + 1e-5) * w["l0.side.norm"]
    assert torch.allclose(streams[0], x, atol=1e-12)
    assert torch.allclose(logits, plain.norm(x, w["final.norm"], 1e-5) @ w["head"].T, atol=1e-12)
    # A second layer reads the next columns of the table.
    two = config([layer("lightning", lightning(1, 2, 2, [0.5]), None)] * 2, width=8, vocab=10, side=3)
    w2 = {n: t.double() for n, t in random_weights(two, 3).items()}
    x = torch.randn(4, 8, dtype=F64, generator=torch.Generator().manual_seed(2))
    e = w2["side.embed"][torch.tensor(tokens), 3:6]
    y = (torch.nn.functional.gelu(x @ w2["l1.side.gate"].T, approximate="tanh") * e) @ w2["l1.side.proj"].T
    assert torch.allclose(plain.token_side(two, w2, 1, x, tokens, 1e-5), plain.norm(y, w2["l1.side.norm"], 1e-5), atol=1e-12)
