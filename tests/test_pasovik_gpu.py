"""The Pasovik decoder through the native engine against the plain implementation (tests/plain_pasovik.py).

Every test builds its own small model.  The engine is driven through its step function (given tokens in, logits out:
what bin/trace_run drives) and through its scheduler (``generate``).  In float32 the engine must agree with the plain
float64 implementation to a few units of 32-bit rounding; in bfloat16 to what rounding the matrix products to 16 bits
costs.  Two cuttings of the same tokens through the engine must agree far closer than either does with the plain
implementation: nothing may depend on portions, batches, pages or slots."""
import copy

import numpy as np
import pytest
import torch

import plain_pasovik as plain
from pasovik_models import CONFIGS, attention, config, dense, latent, layer, lightning, moe, random_weights, write_model

pytestmark = pytest.mark.gpu

TOLERANCE = {"float32": 2e-4, "bfloat16": 6e-2}      # of the logits' root mean square
SAME = {"float32": 2e-5, "bfloat16": 2e-5}           # two cuttings of the same tokens through the engine


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for seed, (name, cfg) in enumerate(CONFIGS.items()):
        w = random_weights(cfg, 20 + seed)
        out[name] = (write_model(tmp_path_factory.mktemp(name), cfg, w), cfg, w)
    return out


def engine(folder, dtype, num_pages=24, page_size=16, max_num_seqs=4, **kw):
    from vosti_amd.engine.native import NativeEngine
    return NativeEngine(folder, dtype=dtype, num_pages=num_pages, page_size=page_size, max_num_seqs=max_num_seqs,
                        enable_prefix_cache=False, graphs=kw.pop("graphs", False), **kw)


def tokens_for(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_cut(eng, rid, tokens, cuts, finish=True):
    """All logits of one request fed in portions of the given sizes."""
    rows, at = [], 0
    for c in cuts:
        rows.append(eng.trace_step([(rid, tokens[at:at + c], list(range(c)))]))
        at += c
    assert at == len(tokens)
    if finish:
        eng.trace_finish(rid)
    return np.concatenate(rows, 0)


def deviation(got, want):
    """Largest row deviation as a fraction of the logits' root mean square."""
    want = np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean(-1)).max() / np.sqrt((want ** 2).mean()))


def close(got, want, dtype):
    """Whether the engine's rows are the plain implementation's.  In float32 every row, to a few units of rounding.  In
    bfloat16 the router sees a rounded input, and where two experts' logits all but tie it may choose the other one: nine
    rows in ten must lie within what rounding costs, and none may be far off."""
    want = np.asarray(want, dtype=np.float64)
    rows = np.sqrt(((got - want) ** 2).mean(-1)) / np.sqrt((want ** 2).mean())
    if dtype == "float32":
        return bool(rows.max() < TOLERANCE[dtype])
    return bool(np.quantile(rows, 0.9) < TOLERANCE[dtype] and rows.max() < 0.5)


def plain_logits(cfg, w, tokens):
    return plain.forward(cfg, w, tokens).numpy()


# ------------------------------------------------------------------------------------------ each mechanism alone
SMALL_MIXER = lightning(1, 4, 4, [0.9])            # a small mixer under the feed-forward that is tested
ALONE = {
    "attention": config([layer("attention", attention(4, 2, 16, 16, rot_dims=8), None)], width=32, vocab=50),
    "attention_whole_head_stretched_and_capped": config([layer("attention", attention(2, 1, 32, 32, rot_dims=32, base=77.0, factor=3.0, softcap=4.0), None)], width=32, vocab=50),
    "attention_wide_values": config([layer("attention", attention(2, 2, 8, 48, rot_dims=4), None)], width=32, vocab=50),
    "attention_keys_wider_than_values": config([layer("attention", attention(3, 3, 40, 24, rot_dims=20, softcap=50.0), None)], width=32, vocab=50),
    "attention_one_head_one_pair": config([layer("attention", attention(1, 1, 16, 16, rot_dims=2, scale=1.0), None)], width=32, vocab=50),
    "attention_many_heads_on_one_key_head": config([layer("attention", attention(24, 1, 16, 16, rot_dims=8), None)], width=32, vocab=50),
    "latent": config([layer("latent_attention", latent(3, 16, 8, 16, kv_rank=24, q_rank=16), None)], width=32, vocab=50),
    "latent_twenty_heads": config([layer("latent_attention", latent(20, 8, 4, 8, kv_rank=16, q_rank=16), None)], width=32, vocab=50),
    "latent_odd_sizes": config([layer("latent_attention", latent(5, 10, 6, 12, kv_rank=13, q_rank=11, base=300.0, factor=2.5), None)], width=32, vocab=50),
    "latent_one_head_wide": config([layer("latent_attention", latent(1, 64, 32, 80, kv_rank=96, q_rank=40), None)], width=32, vocab=50),
    "latent_values_wider_than_the_latent": config([layer("latent_attention", latent(2, 8, 2, 40, kv_rank=8, q_rank=8), None)], width=32, vocab=50),
    "latent_on_the_latent_of_another": config([layer("latent_attention", latent(2, 16, 8, 24, kv_rank=16, q_rank=16), None),
                                               layer("lightning", SMALL_MIXER, None),
                                               layer("latent_attention", latent(4, 8, 8, 8, kv_rank=16, q_rank=24, scale=0.5, kv_from=0), None),
                                               layer("latent_attention", latent(1, 16, 8, 24, kv_rank=16, q_rank=8, kv_from=0), None)], width=32, vocab=50),
    "linear_attention": config([layer("lightning", lightning(4, 8, 16, [0.3, 0.8, 0.95, 1.0]), None)], width=32, vocab=50),
    "linear_attention_one_head": config([layer("lightning", lightning(1, 24, 24, [0.9]), None)], width=32, vocab=50),
    "linear_attention_wide_keys": config([layer("lightning", lightning(2, 100, 40, [0.5, 0.99]), None)], width=32, vocab=50),
    "dense": config([layer("lightning", SMALL_MIXER, dense(52))], width=32, vocab=50),
    "experts": config([layer("lightning", SMALL_MIXER, moe(7, 2, 20, limit=1.0))], width=32, vocab=50),
    "experts_all_chosen": config([layer("lightning", SMALL_MIXER, moe(4, 4, 56, limit=0.6))], width=32, vocab=50),
    "experts_many_of_one": config([layer("lightning", SMALL_MIXER, moe(70, 1, 8))], width=32, vocab=50),
    "side_input": config([layer("lightning", SMALL_MIXER, None), layer("lightning", SMALL_MIXER, dense(8))], width=32, vocab=50, side=8),
    "side_input_of_one_column": config([layer("lightning", SMALL_MIXER, None), layer("attention", attention(1, 1, 16, 16, rot_dims=4), None),
                                        layer("lightning", SMALL_MIXER, None)], width=32, vocab=50, side=1),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ALONE))
def test_each_mechanism_alone(tmp_path, name, dtype):
    cfg = copy.deepcopy(ALONE[name])
    w = random_weights(cfg, 3)
    folder = write_model(tmp_path / name, cfg, w)
    tokens = tokens_for(cfg, 45, 1)
    want = plain_logits(cfg, w, tokens)
    eng = engine(folder, dtype)
    assert close(run_cut(eng, 0, tokens, [45]), want, dtype)
    assert close(run_cut(eng, 1, tokens, [9, 2, 17] + [1] * 17), want, dtype)


def test_many_rows_an_expert_take_the_tile_product(tmp_path):
    """A prompt long enough that the experts' rows go through the grouped tile product, its tokens one by one through the
    other route: the same logits."""
    cfg = config([layer("lightning", SMALL_MIXER, moe(2, 1, 64, limit=1.0))], width=64, vocab=50)
    w = random_weights(cfg, 4)
    folder = write_model(tmp_path / "tiles", cfg, w)
    tokens = tokens_for(cfg, 160, 2)
    for dtype in ("float32", "bfloat16"):
        eng = engine(folder, dtype)
        whole = run_cut(eng, 0, tokens, [160])
        assert close(whole, plain_logits(cfg, w, tokens), dtype)
        assert deviation(run_cut(eng, 1, tokens, [100] + [1] * 60), whole) < SAME[dtype]


def test_a_weight_scales_what_an_expert_reads(tmp_path):
    """Inputs far beyond the experts' limit: the clamps cut w * (W h), so a weight on the output instead would give another
    answer.  The plain implementation's own check first, then the engine against it."""
    cfg = config([layer("lightning", SMALL_MIXER, moe(3, 2, 16, limit=0.25))], width=32, vocab=50)
    w = random_weights(cfg, 6)
    for e in range(3):
        w[f"l0.mlp.e{e}.gate"] = (w[f"l0.mlp.e{e}.gate"].float() * 4).to(torch.bfloat16)
    tokens = tokens_for(cfg, 30, 3)
    h = w["embed"].double()[torch.tensor(tokens)]
    idx, wts = plain.route(cfg["layers"][0]["mlp"], w, "l0.mlp.", h)
    inside = plain.experts(cfg["layers"][0]["mlp"], w, "l0.mlp.", h)
    outside = sum(wts[:, j:j + 1] * torch.stack([plain.expert(w, f"l0.mlp.e{int(idx[t, j])}.", h[t:t + 1], 0.25)[0] for t in range(30)]) for j in range(2))
    assert (inside - outside).abs().max() > 0.05 * inside.abs().max()
    folder = write_model(tmp_path / "weigh", cfg, w)
    for dtype in ("float32", "bfloat16"):
        assert close(run_cut(engine(folder, dtype), 0, tokens, [30]), plain_logits(cfg, w, tokens), dtype)


def test_the_residual_stream_is_32_bit(tmp_path):
    """Sixteen layers with the same weights add the same small update sixteen times to a large embedding; each update is below
    half a step of a 16-bit stream of that size, so a stream that is rounded to 16 bits between sublayers loses them all.
    The plain implementation with such a stream is checked to be far off first; the engine must be near the true one."""
    cfg = config([layer("lightning", SMALL_MIXER, None) for _ in range(16)], width=32, vocab=40)
    w = random_weights(cfg, 5)
    for n in list(w):
        if n.startswith("l0."):
            for i in range(1, 16):
                w[f"l{i}." + n[3:]] = w[n].clone()
    for i in range(16):
        w[f"l{i}.norm1"] = torch.full_like(w[f"l{i}.norm1"], 0.1)
    w["embed"] = (torch.sign(w["embed"].float()) * (32.0 + 16.0 * torch.rand(w["embed"].shape, generator=torch.Generator().manual_seed(1)))).to(torch.bfloat16)
    tokens = tokens_for(cfg, 20, 2)
    want = plain_logits(cfg, w, tokens)
    # The plain layers once more with a stream that is rounded to bfloat16 after every add.
    x = w["embed"].double()[torch.tensor(tokens)]
    for i in range(16):
        y, _ = plain.lightning(cfg["layers"][i]["mixer"], w, f"l{i}.mix.", x, cfg["norm"]["eps"])
        x = (x + plain.norm(y, w[f"l{i}.norm1"], cfg["norm"]["eps"])).to(torch.bfloat16).double()
    lossy = (plain.norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].double().T).numpy()
    assert deviation(lossy, want) > 2.5e-2
    folder = write_model(tmp_path / "deep", cfg, w)
    got = run_cut(engine(folder, "bfloat16"), 0, tokens, [20])
    assert deviation(got, want) < 1.0e-2


# ----------------------------------------------------------------------------- cuttings, batches, pages and slots
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_portions_and_decoding_agree(models, name, dtype):
    folder, cfg, w = models[name]
    n = 150
    tokens = tokens_for(cfg, n, 7)
    want = plain_logits(cfg, w, tokens)
    eng = engine(folder, dtype, page_size=16 if name == "MIXED" else 64)
    whole = run_cut(eng, 0, tokens, [n])
    assert close(whole, want, dtype)
    # The first tokens of a sequence on their own rows (in bfloat16 a router may choose another expert for one of them).
    assert deviation(whole[:4], want[:4]) < (TOLERANCE[dtype] if dtype == "float32" else 0.5)
    cuttings = {
        "token by token": [1] * n,
        "portions down to two tokens": [2, 3, 16, 2, 1, 31, 2, 33, 5, 1, 1, 2, 17, 32, 2],
        "a prompt and then decoding": [n - 60] + [1] * 60,
        "portions that end on page borders": [16, 48, 64, 22],
    }
    for what, cuts in cuttings.items():
        got = run_cut(eng, 1, tokens, cuts)
        assert deviation(got, whole) < SAME[dtype], what


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch(models, dtype):
    """Portions of some requests beside single tokens of others, a request left out of a step, against each alone."""
    folder, cfg, w = models["MIXED"]
    lengths = [70, 23, 41, 5]
    seqs = [tokens_for(cfg, n, 30 + i) for i, n in enumerate(lengths)]
    eng = engine(folder, dtype)
    alone = [run_cut(eng, 10 + i, s, [len(s)]) for i, s in enumerate(seqs)]
    at = [0] * 4
    got = [[] for _ in seqs]
    step = 0
    while any(a < n for a, n in zip(at, lengths)):
        entries, who = [], []
        for i, s in enumerate(seqs):
            if at[i] >= lengths[i] or (step + i) % 5 == 4:        # finished, or left out of this step
                continue
            c = min([7, 1, 2, 1][(step + i) % 4], lengths[i] - at[i])
            entries.append((i, s[at[i]:at[i] + c], list(range(c))))
            who.append((i, c))
            at[i] += c
        step += 1
        if not entries:
            continue
        rows = eng.trace_step(entries)
        r = 0
        for i, c in who:
            got[i].append(rows[r:r + c])
            r += c
    for i in range(4):
        assert deviation(np.concatenate(got[i], 0), alone[i]) < SAME[dtype], i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_and_slots_are_used_again(models, dtype):
    """A pool of one request's pages and one state slot: every request starts in what the one before left."""
    folder, cfg, w = models["MIXED"]
    eng = engine(folder, dtype, num_pages=4, page_size=16, max_num_seqs=1)
    for i, n in enumerate([60, 17, 64, 33]):
        tokens = tokens_for(cfg, n, 50 + i)
        got = run_cut(eng, i, tokens, [n // 2, n - n // 2 - 3, 1, 1, 1])
        assert close(got, plain_logits(cfg, w, tokens), dtype), i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(models, dtype):
    folder, cfg, w = models["MIXED"]
    n = 300
    tokens = tokens_for(cfg, n, 9)
    eng = engine(folder, dtype, num_pages=20)
    got = run_cut(eng, 0, tokens, [40] + [1] * (n - 40))
    assert close(got, plain_logits(cfg, w, tokens), dtype)


# ------------------------------------------------------------------------- a key that stands out, wherever it is put
def marked_model(kind, head=16):
    """One layer whose attention has one head whose query is a constant direction and whose key lies along it for one
    token alone, the mark (token 1), and whose value carries the mark into the logits: the logits at a position move if and
    only if the marked key is at that position or before it.  kind: "attention", "latent", or "latent reader" (the first
    layer's output is switched off and a second layer reads the first layer's latent)."""
    if kind == "attention":
        layers = [layer("attention", attention(1, 1, head, head, rot_dims=2, base=1e6, scale=1.0), None)]
    else:
        layers = [layer("latent_attention", latent(1, head, 2, head, kv_rank=16, q_rank=8, base=1e6, scale=1.0), None)]
        if kind == "latent reader":
            layers.append(layer("latent_attention", latent(1, head, 2, head, kv_rank=16, q_rank=8, base=1e6, scale=1.0, kv_from=0), None))
    cfg = config(layers, width=32, vocab=12)
    w = random_weights(cfg, 77)
    W = cfg["width"]
    embed = torch.zeros(12, W)
    embed[:, 0] = 1.0                      # every token: a constant channel that makes the query
    embed[1, 1] = 6.0                      # the mark: a channel that makes the key and the value
    embed[2:, 2:] = torch.randn(10, W - 2, generator=torch.Generator().manual_seed(3)) * 0.2
    w["embed"] = embed.to(torch.bfloat16)
    bf = torch.bfloat16
    for i in range(len(layers)):
        p = f"l{i}.mix."
        w[f"l{i}.norm1"] = torch.ones(W).to(bf)
        if kind == "attention":
            q, k, v = torch.zeros(head, W), torch.zeros(head, W), torch.zeros(head, W)
            q[head - 1, 0] = 1.0           # the last dimension of the head is not rotated; the head norm makes it sqrt(head)
            k[head - 1, 1] = 1.0           # a key's last dimension: sqrt(head) for the mark, 0 for any other token
            v[:, 1] = 1.0
            w[p + "q"], w[p + "k"], w[p + "v"] = q.to(bf), k.to(bf), v.to(bf)
            w[p + "q.norm"], w[p + "k.norm"] = torch.ones(head).to(bf), torch.ones(head).to(bf)
        else:
            dq, uq = torch.zeros(8, W), torch.zeros(head + 2, 8)
            dq[0, 0] = 1.0                 # the query's latent: sqrt(8) in its first entry for every token
            uq[0, 0] = 3.0                 # q_flat's first entry
            w[p + "dq"], w[p + "uq"], w[p + "dq.norm"] = dq.to(bf), uq.to(bf), torch.ones(8).to(bf)
            if i == 0:
                dkv = torch.zeros(18, W)
                dkv[0, 1] = 1.0            # the latent's first entry: the mark
                dkv[1, 0] = 1.0            # its second: the constant, so that its norm never divides by nothing
                w[p + "dkv"], w[p + "dkv.norm"] = dkv.to(bf), torch.ones(16).to(bf)
            uk, uv = torch.zeros(head, 16), torch.zeros(head, 16)
            uk[0, 0] = 1.0                 # the key's first entry is the latent's first
            uv[:, 0] = 1.0
            w[p + "uk"], w[p + "uv"] = uk.to(bf), uv.to(bf)
            w[p + "g"] = torch.zeros(head, W).to(bf)        # every gate is one half
    if kind == "latent reader":
        w["l0.norm1"] = torch.zeros(W).to(bf)               # the first layer adds nothing
    return cfg, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "latent", "latent reader"])
def test_a_marked_key_is_seen_from_its_own_position_on(tmp_path, dtype, kind):
    page = 16
    cfg, w = marked_model(kind)
    folder = write_model(tmp_path / "marked", cfg, w)
    eng = engine(folder, dtype, num_pages=60, page_size=page)
    n = 100
    rid = 0
    # (marked position, asking position): the mark at the asking position, just before and just after it, at page borders,
    # the first tokens, far away.
    cases = [(0, 0), (1, 0), (0, 1), (0, 99), (1, 99), (40, 40), (41, 40), (40, 41), (31, 32), (32, 31), (32, 32), (47, 48), (48, 47), (15, 16), (16, 15),
             (5, 95), (95, 95), (96, 95), (99, 98), (63, 64), (64, 63)]
    for mark, ask in cases:
        tokens = [2 + (i * 7) % 10 for i in range(n)]
        base = list(tokens)
        tokens[mark] = 1
        visible = mark <= ask
        p_marked = plain_logits(cfg, w, tokens)[ask]
        p_base = plain_logits(cfg, w, base)[ask]
        moved = np.abs(p_marked - p_base).max()
        assert (moved > 0.05) == visible, (mark, ask, moved)        # the plain implementation itself, first
        for cuts in ([n], [ask] + [1] * (n - ask) if ask else [n], [mark + 1, n - mark - 1] if mark + 1 < n else [n], [3, 2] + [5] * 19):
            got = run_cut(eng, rid, tokens, cuts)[ask]
            rid += 1
            assert np.sqrt(((got - p_marked) ** 2).mean()) < TOLERANCE[dtype] * np.sqrt((p_marked ** 2).mean()) + 1e-3, (mark, ask, cuts[:3])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "latent"])
def test_a_marked_key_far_away_among_hundreds(tmp_path, dtype, kind):
    """One key 900 tokens back, over many pages and segments, in a prompt, in portions and in decoding."""
    cfg, w = marked_model(kind)
    folder = write_model(tmp_path / "far", cfg, w)
    n = 1000
    tokens = [2 + (i * 7) % 10 for i in range(n)]
    tokens[70] = 1
    want = plain_logits(cfg, w, tokens)[-40:]
    base = list(tokens)
    base[70] = 5
    assert np.abs(want - plain_logits(cfg, w, base)[-40:]).max() > 0.05
    eng = engine(folder, dtype, num_pages=70, page_size=16)
    for rid, cuts in enumerate(([n], [n - 40] + [1] * 40, [333, 2, 400, 225] + [1] * 40)):
        got = run_cut(eng, rid, tokens, cuts)[-40:]
        assert deviation(got, want) < TOLERANCE[dtype] + 1e-3, cuts[:3]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_capped_scores(tmp_path, dtype):
    """Scores far beyond the cap: without it one key would take all the weight."""
    cfg, w = marked_model("attention")
    cfg["layers"][0]["mixer"]["softcap"] = 1.5
    # Values that differ from token to token: the layer's norm takes the output's size away, so the cap must show in its direction.
    w["l0.mix.v"] = torch.randn(16, 32, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    folder = write_model(tmp_path / "cap", cfg, w)
    tokens = [2 + (i * 7) % 10 for i in range(40)]
    tokens[3] = 1
    want = plain_logits(cfg, w, tokens)
    free = copy.deepcopy(cfg)
    del free["layers"][0]["mixer"]["softcap"]
    assert np.abs(want - plain_logits(free, w, tokens)).max() > 0.05
    assert close(run_cut(engine(folder, dtype), 0, tokens, [40]), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_recurrence_cut_between_any_two_tokens(tmp_path, dtype):
    cfg = config([layer("lightning", lightning(2, 16, 16, [0.7, 0.98]), None), layer("lightning", lightning(4, 8, 24, [0.1, 0.5, 0.9, 0.999]), moe(4, 2, 16))],
                 width=32, vocab=50, side=3)
    w = random_weights(cfg, 8)
    folder = write_model(tmp_path / "cuts", cfg, w)
    n = 40
    tokens = tokens_for(cfg, n, 4)
    eng = engine(folder, dtype)
    whole = run_cut(eng, 0, tokens, [n])
    assert close(whole, plain_logits(cfg, w, tokens), dtype)
    for cut in range(1, n):
        assert deviation(run_cut(eng, cut, tokens, [cut, n - cut]), whole) < SAME[dtype], cut


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slow_decay_remembers_the_first_token(tmp_path, dtype):
    """A decay near one keeps the first token's key and value for hundreds of tokens: a state that is lost or reset on the
    way shows in the last logits."""
    cfg = config([layer("lightning", lightning(1, 8, 8, [0.9995]), None)], width=32, vocab=20)
    w = random_weights(cfg, 12)
    w["embed"][0] = (w["embed"][0].float() * 30).to(torch.bfloat16)      # a first token that is hard to forget
    folder = write_model(tmp_path / "slow", cfg, w)
    n = 260
    a = [0] + [1 + t % 19 for t in tokens_for(cfg, n - 1, 5)]
    b = list(a)
    b[0] = 1
    want_a, want_b = plain_logits(cfg, w, a), plain_logits(cfg, w, b)
    assert np.abs(want_a[-1] - want_b[-1]).max() > 0.01          # the plain implementation: the first token still matters
    eng = engine(folder, dtype, num_pages=20)
    for tokens, want in ((a, want_a), (b, want_b)):
        assert close(run_cut(eng, 0, tokens, [100, 7] + [1] * (n - 107)), want, dtype)


# ------------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(models, graphs):
    """create_engine -> the scheduler, the step function, the sampler: the tokens are the plain implementation's."""
    from vosti_amd.engine import create_engine
    from vosti_amd.sampling.params import SamplingParams
    folder, cfg, w = models["MIXED"]
    prompts = [tokens_for(cfg, n, 60 + i) for i, n in enumerate([19, 3, 40])]
    eng = create_engine(folder, dtype="float32", num_pages=24, page_size=16, max_num_seqs=4, graphs=graphs)
    out = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for prompt, got in zip(prompts, out):
        assert list(got) == plain.generate_greedy(cfg, w, prompt, 12)


def test_the_command_line_generates_the_plain_tokens(models):
    """The engine's program, started as a user starts it with --family pasovik: greedy tokens of the plain implementation."""
    import json
    import subprocess
    from vosti_amd.kernels import build
    folder, cfg, w = models["MIXED"]
    program = str(build.ensure("engine", verbose=False))
    lib = build.ensure("f32", verbose=False)
    prompt = tokens_for(cfg, 21, 70)
    r = subprocess.run([program, "--family", "pasovik", "--dtype", "float32", "--lib-dir", str(lib.parent), "--model-path", str(folder),
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8", "--page-size", "16"], capture_output=True, text=True, timeout=110, env={})
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads([l for l in r.stdout.splitlines() if l.startswith("MODEL_OUTPUT_TOKEN_IDS=")][0].split("=", 1)[1])
    assert out == plain.generate_greedy(cfg, w, prompt, 8)


# --------------------------------------------------------------------------------------------- the replay program
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program_with_four_slots_and_a_pool_for_the_live_requests(models, tmp_path, dtype):
    """bin/trace_run as a user starts it: six requests of which at most four are live, portions of prompts beside single
    tokens, requests left out of steps, a pool sized for the live requests alone (so that pages and state slots are used
    again), a name that comes back after its request ended.  Every row against the plain implementation."""
    import json
    import random
    import subprocess
    import sys
    from pathlib import Path
    folder, cfg, w = models["MIXED"]
    lengths = {"a": 70, "b": 33, "c": 150, "d": 9, "e": 64, "f": 101, "a again": 41}
    tokens = {name: tokens_for(cfg, n, 80 + i) for i, (name, n) in enumerate(lengths.items())}
    rng = random.Random(5)
    waiting, live, fed, steps, most = list(lengths), [], {}, [], 0
    while waiting or live:
        while waiting and len(live) < 4 and not (waiting[0] == "a again" and "a" in live):
            live.append(waiting.pop(0))
            fed[live[-1]] = 0
        most = max(most, sum(-(-lengths[n] // 64) * 64 for n in live))
        entries, end = [], []
        for name in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                                            # left out of this step
            left = lengths[name] - fed[name]
            size = min(left, 1 if left <= 6 else rng.choice([1, 2, 3, 7, 16, 40]))
            entries.append({"id": name.split()[0], "name": name, "tokens": tokens[name][fed[name]:fed[name] + size], "want": list(range(size))})
            fed[name] += size
            if fed[name] == lengths[name]:
                end.append(name.split()[0])
                live.remove(name)
        steps.append({"step": len(steps), "entries": entries, "end": end})
    cmd = [sys.executable, str(Path(__file__).resolve().parent.parent / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
           "--out", str(tmp_path), "--max-tokens", str(most)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for rec in steps:
        proc.stdin.write(json.dumps(rec) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == f"done {rec['step']}"
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    rows = {name: [] for name in lengths}
    for rec in steps:
        if not any(e["want"] for e in rec["entries"]):
            continue
        got = np.fromfile(tmp_path / f"{rec['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        at = 0
        for e in rec["entries"]:
            rows[e["name"]].append(got[at:at + len(e["want"])])
            at += len(e["want"])
        assert at == got.shape[0]
    for name in lengths:
        assert close(np.concatenate(rows[name], 0), plain_logits(cfg, w, tokens[name]), dtype), name
