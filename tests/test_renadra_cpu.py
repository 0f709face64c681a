"""Renadra without a GPU: its configuration reader and the specification built from it, the order in which layers run,
the tensor names a checkpoint must hold, the pages of kept first positions in the cache manager, and the plain
implementation's mechanisms against closed forms of the same sums written out another way."""

import copy
import math

import pytest
import torch

from tests.renadra_configs import ALONE, RENA_A, RENA_B, RENA_C, left
from tests.plain import renadra_plain as plain


def build(cfg):
    from paged_llm_amd.config.registry import lookup_architecture
    from paged_llm_amd.models.decoder import DecoderModel
    arch = lookup_architecture(cfg)
    spec = arch.build_spec(arch.read_config(cfg))
    return spec, DecoderModel(spec, torch.float32, "cpu", max_positions=64)


def test_architecture_is_registered():
    from paged_llm_amd.config.registry import lookup_architecture
    assert lookup_architecture(RENA_A).name == "Renadra"


def test_repeated_layers_are_steps_of_one_layer_with_a_cache_or_state_each():
    spec, model = build(RENA_A)
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 1, 2, 1, 2, 3] and len(spec.layers) == 4
    assert [s.entry for s in spec.schedule] == [None, None, None, 0, None, 0, None, None]       # the embedding is added in front of passes two and three
    assert plain.run_order(RENA_A) == [(s.layer, s.entry is not None) for s in spec.schedule]
    states = model.state_specs()
    assert sorted(k for k in states if k != "embedding") == [0, 1, 3, 5, 7]
    assert states["embedding"].shape == (1,) and states["embedding"].dtype == torch.int32
    assert states[0].shape == (3 * 20 * 24,) and states[1].shape == (3 * 20 * 24,) and states[7].shape == (2 * 16 * 40,)
    groups = list(model.cache_groups().values())
    assert sorted(sorted(g.owners) for g in groups) == [[1, 3, 5], [2, 4, 6]]
    by_owner = {tuple(sorted(g.owners)): g.spec for g in groups}
    assert (by_owner[(1, 3, 5)].kind, by_owner[(1, 3, 5)].window, by_owner[(1, 3, 5)].keep_first) == ("window", 21, 3)
    assert (by_owner[(2, 4, 6)].kind, by_owner[(2, 4, 6)].window, by_owner[(2, 4, 6)].keep_first) == ("window", 21, 0)
    names = set(model.weight_specs())
    assert {"embed", "bigram", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q", "l0.mix.f", "l0.mix.f.b", "l0.mix.lower", "l0.mix.v",
            "l0.mix.norm", "l0.mix.o", "l0.mlp.gate", "l0.mlp.up", "l0.mlp.down", "l1.mix.left.q", "l1.mix.left.q.b", "l1.mix.left.k",
            "l1.mix.left.k.b", "l1.mix.left.pb", "l1.mix.left.o", "l1.mix.right.q", "l1.mix.right.k", "l1.mix.right.v", "l1.mix.right.g",
            "l1.mix.right.norm", "l1.mix.right.o", "l2.mix.q", "l2.mix.q.b", "l2.mix.k.b", "l2.mix.v", "l2.mix.v.b", "l2.mix.o", "l2.mix.o.b"} <= names
    assert not {"l1.mix.left.v", "l1.mix.left.v.b", "l1.mix.left.o.b", "l2.norm2", "l2.mlp.gate", "l0.mix.k", "l2.mix.pb", "l4.norm1", "loop"} & names


def test_sizes_come_from_the_configuration():
    _, model = build(RENA_B)
    specs = model.weight_specs()
    assert specs["bigram"].shape == (1010, 50) and specs["embed"].shape == (77, 50)
    assert specs["l0.mix.q"].shape == (30, 50) and specs["l0.mix.v"].shape == (18, 50) and specs["l0.mix.o"].shape == (50, 18)
    assert specs["l1.mix.left.q"].shape == (30, 50) and specs["l1.mix.left.k"].shape == (30, 50) and specs["l1.mix.left.pb"].shape == (3,)
    assert specs["l1.mix.right.q"].shape == (140, 50) and specs["l1.mix.right.v"].shape == (132, 50) and specs["l1.mix.right.norm"].shape == (132,)
    assert specs["l2.mix.q"].shape == (70, 50) and specs["l2.mix.lower"].shape == (70,) and specs["l2.mix.norm"].shape == (66,)
    assert "l1.norm2" not in specs and specs["l2.mlp.down"].shape == (50, 34)
    assert model.state_specs()[1].shape == (2 * 70 * 66,) and model.state_specs()[2].shape == (70 * 66,)
    assert not model.spec.stream_ops and all(s.entry is None for s in model.spec.schedule)
    spec, model = build(RENA_C)
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 0, 1, 2] and [s.entry for s in spec.schedule] == [None, None, None, 0, None, None]
    keeps = sorted(g.spec.keep_first for g in model.cache_groups().values())
    assert keeps == [0, 0, 2]


def test_bad_configurations_are_refused():
    from paged_llm_amd.config.registry import lookup_architecture
    arch = lookup_architecture(RENA_A)
    for change in (lambda c: c["layers"][0].update(type="mamba"), lambda c: c["layers"][0]["mlp"].update(kind="moe"),
                   lambda c: c.update(loop={"start": 2, "stop": 2, "times": 2}), lambda c: c.update(loop={"start": 0, "stop": 9, "times": 2}),
                   lambda c: c["embedding"]["bigram"].update(buckets=0)):
        bad = copy.deepcopy(RENA_A)
        change(bad)
        with pytest.raises(ValueError):
            arch.read_config(bad)
    bad = copy.deepcopy(RENA_A)
    bad["layers"][1]["mixer"]["left"]["vdim"] = 8                    # values that are the keys have the keys' size
    with pytest.raises(ValueError):
        build(bad)
    bad = copy.deepcopy(RENA_A)
    bad["layers"][1]["mixer"]["right"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        build(bad)


def test_rotary_tables_of_the_engine_are_the_plain_ones():
    from paged_llm_amd.parts.registry import BuildEnv
    from paged_llm_amd.parts.rope import RotaryEncoding
    env = BuildEnv(64, torch.float32, torch.device("cpu"), 64, shared={})
    for dims, base, scaling in ((16, 1e4, {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}), (40, 100.0, {"factor": 6.0, "original": 512, "fast": 24.0, "slow": 1.5}),
                                (16, 5e5, {"factor": 16.0, "original": 32, "fast": 4.0, "slow": 0.5}), (10, 33.0, None)):
        engine_scaling = dict(scaling, rope_type="yarn") if scaling else None
        part = RotaryEncoding({"head_dim": 48, "theta": base, "rotary_dim": dims, "scaling": engine_scaling, "exact_frequencies": True}, env)
        f, mag = plain.frequencies(dims, base, scaling)
        assert torch.equal(part.inverse_frequencies(), f.to(torch.float32))
        assert part.table_factor() == mag and (mag > 1.0) == bool(scaling)
        part.prepare(50)
        angles = torch.arange(50, dtype=torch.float64)[:, None] * f[None, :]
        assert float((part.cos.double() - angles.cos() * mag).abs().max()) < 2e-5 and float((part.sin.double() - angles.sin() * mag).abs().max()) < 2e-5
    # the three ranges of the blend: pairs below lo as they are, pairs above hi divided by the factor, a ramp between
    f, _ = plain.frequencies(16, 1e4, {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0})
    plain_f, _ = plain.frequencies(16, 1e4, None)
    ratio = (f / plain_f).tolist()
    assert ratio[0] == 1.0 and ratio[-1] == 0.25 and any(0.25 < r < 1.0 for r in ratio) and ratio == sorted(ratio, reverse=True)


def test_bigram_rows():
    assert plain.bigram_rows([4, 9, 9, 0], 61, 5, 3) == [61, (4 * 5 + 9 * 3) % 61, (9 * 5 + 9 * 3) % 61, (9 * 5) % 61]
    table, pairs = torch.arange(20.0).reshape(10, 2), torch.arange(16.0).reshape(8, 2) * 100
    x = plain.embedding([3, 1], table, pairs, 0.5, {"buckets": 7, "mul_prev": 2, "mul_cur": 3})
    assert torch.equal(x, torch.stack([table[3] * 0.5 + pairs[7], table[1] * 0.5 + pairs[(3 * 2 + 1 * 3) % 7]]))


def test_visible_keys():
    see = plain.visible(12, 4, 2)
    for i in range(12):
        for j in range(12):
            assert bool(see[i, j]) == (j <= i and (i - j < 4 or j < 2))
    assert int(plain.visible(12, 1, 0).sum()) == 12 and int(plain.visible(5, 0, 0).sum()) == 15


def test_sigmoid_attention_token_by_token():
    """Against a loop over queries and visible keys with the weights written out."""
    torch.manual_seed(0)
    m = left(heads=4, kv_heads=2, dim=8, size=5, keep_first=2, rot_dims=4, base=50.0, scale=0.4, softcap=3.0, scaling={"factor": 2.0, "original": 8, "fast": 2.0, "slow": 0.5})
    T, W = 14, 16
    w = {"q": torch.randn(32, W), "q.b": torch.randn(32), "k": torch.randn(16, W), "k.b": torch.randn(16), "pb": torch.randn(4), "o": torch.randn(W, 32)}
    h = torch.randn(T, W, dtype=torch.float64)
    w = {k: v.double() for k, v in w.items()}
    got = plain.sigmoid_attention(h, w, m, list(range(T)))
    q = (h @ w["q"].T + w["q.b"]).view(T, 4, 8)
    k = (h @ w["k"].T + w["k.b"]).view(T, 2, 8)
    rq, rk = plain.rotate(q, range(T), 4, 50.0, False, m["rot"]["scaling"]), plain.rotate(k, range(T), 4, 50.0, False, m["rot"]["scaling"])
    out = torch.zeros(T, 4, 8, dtype=torch.float64)
    for i in range(T):
        for head in range(4):
            for j in range(i + 1):
                if i - j < 5 or j < 2:
                    s = 3.0 * math.tanh(float(rq[i, head] @ rk[j, head // 2]) * 0.4 / 3.0)
                    out[i, head] += k[j, head // 2] / (1.0 + math.exp(-(s + float(w["pb"][head]))))       # the value is the key before its rotation
    assert float((got - out.reshape(T, 32) @ w["o"].T).abs().max()) < 1e-9
    # the rotation leaves the elements behind the rotated width alone and scales the rotated pairs' length by the tables' factor
    assert torch.equal(rq[..., 4:], q[..., 4:])
    mag = plain.frequencies(4, 50.0, m["rot"]["scaling"])[1]
    assert float(((rq[..., :4] ** 2).sum(-1) - mag * mag * (q[..., :4] ** 2).sum(-1)).abs().max()) < 1e-9


def test_windowed_attention_norms_its_values():
    torch.manual_seed(1)
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 6, "mask": {"size": 3}, "rot": {"base": 10.0, "dims": 4}, "scale": 0.5}
    T, W = 9, 8
    w = {k: v.double() for k, v in {"q": torch.randn(8, W), "q.b": torch.randn(8), "k": torch.randn(4, W), "k.b": torch.randn(4), "v": torch.randn(6, W),
                                    "v.b": torch.randn(6), "o": torch.randn(W, 12), "o.b": torch.randn(W)}.items()}
    h = torch.randn(T, W, dtype=torch.float64)
    got = plain.attention(h, w, m, 1e-3, list(range(T)))
    q, k = (h @ w["q"].T + w["q.b"]).view(T, 2, 4), (h @ w["k"].T + w["k.b"]).view(T, 1, 4)
    v = h @ w["v"].T + w["v.b"]
    v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-3)
    rq, rk = plain.rotate(q, range(T), 4, 10.0, True), plain.rotate(k, range(T), 4, 10.0, True)
    # interleaved pairs: elements (0, 1) turn by the first frequency
    a = 3 * 1.0
    assert abs(float(rq[3, 0, 0]) - (float(q[3, 0, 0]) * math.cos(a) - float(q[3, 0, 1]) * math.sin(a))) < 1e-12
    out = torch.zeros(T, 2, 6, dtype=torch.float64)
    for i in range(T):
        for head in range(2):
            js = [j for j in range(i + 1) if i - j < 3]
            p = torch.softmax(torch.stack([rq[i, head] @ rk[j, 0] * 0.5 for j in js]), 0)
            out[i, head] = sum(p[n] * v[j] for n, j in enumerate(js))
    assert float((got - (out.reshape(T, 12) @ w["o"].T + w["o.b"])).abs().max()) < 1e-9


def test_recurrences_against_the_sums_over_earlier_tokens():
    torch.manual_seed(2)
    T, W, H, N, P = 11, 8, 2, 3, 5
    h = torch.randn(T, W, dtype=torch.float64)
    # hgrn2: o_t = sum_s (prod_{s < r <= t} f_r) * (1 - f_s) * q_t  . v_s, channel by channel
    w = {k: v.double() for k, v in {"q": torch.randn(H * N, W), "f": torch.randn(H * N, W), "f.b": torch.randn(H * N), "lower": torch.rand(H * N),
                                    "v": torch.randn(H * P, W), "norm": torch.rand(P) + 0.5, "o": torch.randn(W, H * P)}.items()}
    got = plain.hgrn2(h, w, {"heads": H, "dim": N, "vdim": P}, 1e-4)
    q = plain.silu(h @ w["q"].T).view(T, H, N)
    f = (w["lower"] + (1 - w["lower"]) * torch.sigmoid(h @ w["f"].T + w["f.b"])).view(T, H, N)
    assert bool((f >= w["lower"].view(H, N)).all()) and bool((f < 1).all())
    v = (h @ w["v"].T).view(T, H, P)
    o = torch.zeros(T, H, P, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            carry = torch.ones(H, N, dtype=torch.float64)
            for r in range(s + 1, t + 1):
                carry = carry * f[r]
            o[t] += ((q[t] * carry * (1 - f[s])).sum(-1, keepdim=True)) * v[s]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-4) * w["norm"]
    assert float((got - o.reshape(T, H * P) @ w["o"].T).abs().max()) < 1e-9
    # lightning: o_t = sum_s decay^(t - s) (q_t . k_s) v_s, all heads normed together
    decay = [0.7, 0.95]
    w = {k: v.double() for k, v in {"q": torch.randn(H * N, W), "k": torch.randn(H * N, W), "v": torch.randn(H * P, W), "g": torch.randn(H * P, W),
                                    "norm": torch.rand(H * P) + 0.5, "o": torch.randn(W, H * P)}.items()}
    got = plain.lightning_attention(h, w, {"heads": H, "dim": N, "vdim": P, "decay": decay}, 1e-4)
    q, k, v = (plain.silu(h @ w[n].T).view(T, H, -1) for n in ("q", "k", "v"))
    o = torch.zeros(T, H, P, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            for head in range(H):
                o[t, head] += decay[head] ** (t - s) * float(q[t, head] @ k[s, head]) * v[s, head]
    o = o.reshape(T, H * P)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-4) * w["norm"] * torch.sigmoid(h @ w["g"].T)
    assert float((got - o @ w["o"].T).abs().max()) < 1e-9


def _random_weights(cfg, seed=0):
    from paged_llm_amd.weights.random_init import _declared_weights, draw_weights
    return dict(draw_weights(_declared_weights(cfg), seed, torch.float32, std=cfg["width"] ** -0.5, norm_jitter=True))


def test_the_whole_model_is_the_sum_of_its_branches():
    """The stream after every layer run, rebuilt from the mechanisms one by one: the embedding added in front of the later
    passes of the repeated range, the two sides of a parallel mixer with their factors, layers without a feed-forward."""
    cfg = RENA_A
    w = {k: t.double() for k, t in _random_weights(cfg).items()}
    toks = [7, 1, 250, 33, 33, 9, 120, 5, 64]
    outs = []
    logits = plain.forward(cfg, w, toks, torch.float64, outs)
    eps = cfg["norm"]["eps"]
    x0 = plain.embedding(toks, w["embed"], w["bigram"], cfg["embedding"]["scale"], cfg["embedding"]["bigram"])
    x, n = x0.clone(), 0
    for i, again in plain.run_order(cfg):
        if again:
            x = x + x0
        layer = cfg["layers"][i]
        h = plain.rms_norm(x, w[f"l{i}.norm1"], eps)
        wm = {k[len(f"l{i}.mix."):]: t for k, t in w.items() if k.startswith(f"l{i}.mix.")}
        if layer["type"] == "parallel":
            m = layer["mixer"]
            a = m["left_scale"] * plain.sigmoid_attention(h, {k[5:]: t for k, t in wm.items() if k.startswith("left.")}, m["left"], range(len(toks))) \
                + m["right_scale"] * plain.lightning_attention(h, {k[6:]: t for k, t in wm.items() if k.startswith("right.")}, m["right"], eps)
        elif layer["type"] == "attention":
            a = plain.attention(h, wm, layer["mixer"], eps, range(len(toks)))
        else:
            a = plain.hgrn2(h, wm, layer["mixer"], eps)
        x = x + a
        if layer["mlp"]:
            x = x + plain.gated_mlp(plain.rms_norm(x, w[f"l{i}.norm2"], eps), {k[len(f"l{i}.mlp."):]: t for k, t in w.items() if k.startswith(f"l{i}.mlp.")})
        assert float((outs[n] - x).abs().max()) < 1e-9
        n += 1
    assert n == 8 and float((logits - plain.rms_norm(x, w["final.norm"], eps) @ w["head"].T).abs().max()) < 1e-9
    # a later token never changes an earlier row, and the first token takes the bigram table's last row
    shorter = plain.forward(cfg, w, toks[:4], torch.float64)
    assert float((shorter - logits[:4]).abs().max()) < 1e-9
    moved = dict(w, bigram=w["bigram"].clone())
    moved["bigram"][-1] += 1.0
    assert float((plain.forward(cfg, moved, toks, torch.float64)[0] - logits[0]).abs().max()) > 1e-3


def test_every_alone_configuration_builds():
    for cfg in ALONE.values():
        spec, model = build(cfg)
        assert set(_random_weights(cfg)) == set(model.weight_specs())


# --------------------------------------------------------------------------- pages of kept first positions
def test_pages_of_the_kept_first_positions_stay_while_the_window_moves_on():
    from paged_llm_amd.cache.block_manager import NO_PAGE, CacheManager, GroupSpec
    m = CacheManager([GroupSpec("win", "window", 6, keep_first=5)], 6, 4, False)       # pages of 4 positions: the kept ones take two
    assert m.allocate("a", 0, 10)
    at = 10
    for _ in range(60):
        assert m.allocate("a", at, 1), at
        at += 1
        table = m.block_table("a", "win")
        assert table[0] != NO_PAGE and table[1] != NO_PAGE
        first_key = at - 1 - 6 + 1
        assert all(p != NO_PAGE for p in table[first_key // 4:])
        assert all(p == NO_PAGE for p in table[2:first_key // 4])
        assert len([p for p in table if p != NO_PAGE]) <= 2 + 3
    m.check_invariants()
    m.free("a")
    assert m.num_free_pages("win") == 6
    # a request that enters with a long portion holds the kept pages and those of the window's end, and none between
    assert m.allocate("b", 0, 3) and m.allocate("b", 3, 20)
    table = m.block_table("b", "win")
    assert table[0] != NO_PAGE and table[1] != NO_PAGE and len(table) == 6
    with pytest.raises(ValueError):
        GroupSpec("full", "full", 0, keep_first=3)
