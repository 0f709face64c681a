"""Nesezen without a GPU: its configuration reader and the specification built from it, the order in which layers run,
the tensor names a checkpoint must hold, and the plain implementation's mechanisms against closed forms of the same
sums written out another way."""

import copy
import math

import pytest
import torch

from tests.nesezen_configs import ALONE, NESE_A, NESE_B, NESE_C
from tests.plain import nesezen_plain as plain


def build(cfg):
    from paged_llm_amd.config.registry import lookup_architecture
    from paged_llm_amd.models.decoder import DecoderModel
    arch = lookup_architecture(cfg)
    spec = arch.build_spec(arch.read_config(cfg))
    return spec, DecoderModel(spec, torch.float32, "cpu", max_positions=64)


def test_architecture_is_registered():
    from paged_llm_amd.config.registry import lookup_architecture
    assert lookup_architecture(NESE_A).name == "Nesezen"


def test_borrowed_weights_are_steps_of_one_layer_with_a_cache_or_state_each():
    spec, model = build(NESE_A)
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 0, 1, 2] and len(spec.layers) == 3
    # the two runs of the matrix memory own a state each: S with the normaliser as a last column, and the maxima behind it
    assert sorted(model.state_specs()) == [1, 4]
    assert model.state_specs()[1].shape == (3 * 20 * (24 + 1) + 3,)
    groups = list(model.cache_groups().values())
    assert sorted(sorted(g.owners) for g in groups) == [[0, 3], [2, 5]]
    by_owner = {tuple(sorted(g.owners)): g.spec for g in groups}
    assert (by_owner[(0, 3)].kind, by_owner[(0, 3)].window) == ("window", 21) and by_owner[(2, 5)].kind == "full"
    names = set(model.weight_specs())
    assert {"embed", "head", "final.norm", "final.norm.b", "final.norm.alpha", "l0.norm1", "l0.norm1.b", "l0.norm1.alpha", "l0.norm2.alpha",
            "l0.mix.q", "l0.mix.o", "l0.mlp.gate", "l0.mlp.down", "l1.mix.i", "l1.mix.f.b", "l1.mix.norm", "l1.mix.g", "l1.mlp.router",
            "l1.mlp.e5.down", "l1.mlp.shared.up", "l1.mlp.shared.sg", "l2.mix.dq", "l2.mix.dq.norm", "l2.mix.uq", "l2.mix.dkv", "l2.mix.dkv.norm",
            "l2.mix.uk", "l2.mix.uv", "l2.mix.g", "l2.mix.o"} <= names
    assert not {"l3.norm1", "l4.mix.q", "l5.mix.dq", "l2.norm2", "l2.mlp.gate", "l1.mlp.e6.gate", "l1.mlp.correction", "l0.mix.g", "l2.mix.q"} & names


def test_sizes_come_from_the_configuration():
    _, model = build(NESE_B)
    specs = model.weight_specs()
    assert specs["l0.mix.dq"].shape == (12, 50) and specs["l0.mix.uq"].shape == (5 * 6, 12) and specs["l0.mix.uk"].shape == (30, 20)
    assert specs["l0.mix.uv"].shape == (50, 20) and specs["l0.mix.g"].shape == (5, 50) and specs["l0.mix.o"].shape == (50, 50)
    assert specs["l0.mlp.router"].shape == (3, 50) and "l0.mlp.shared.gate" not in specs and "l0.mlp.e3.gate" not in specs
    assert specs["l1.mix.q"].shape == (140, 50) and specs["l1.mix.v"].shape == (132, 50) and specs["l1.mix.i"].shape == (2, 50)
    assert specs["l1.mix.i.b"].shape == (2,) and specs["l1.mix.norm"].shape == (132,)
    assert specs["l2.mix.q"].shape == (30, 50) and specs["l2.mix.v"].shape == (18, 50) and specs["l2.mix.o"].shape == (50, 18)
    assert specs["l2.mlp.shared.sg"].shape == (1, 50) and specs["l2.mlp.shared.down"].shape == (50, 18) and specs["l2.mlp.e3.up"].shape == (10, 50)
    assert specs["final.norm.alpha"].shape == ()
    assert model.state_specs()[1].shape == (2 * 70 * 67 + 2,)
    _, model = build(NESE_C)
    assert sorted(model.state_specs()) == [3] and "l3.norm2" not in model.weight_specs() and "l0.norm2" not in model.weight_specs()


def test_bad_configurations_are_refused():
    from paged_llm_amd.config.registry import lookup_architecture
    arch = lookup_architecture(NESE_A)
    for change in (lambda c: c["layers"][0].update(type="conv"), lambda c: c["layers"][0]["mlp"].update(kind="sparse"),
                   lambda c: c["layers"][3].update(weights_of=4), lambda c: c["layers"][3].update(weights_of=1), lambda c: c.update(vocab=0)):
        cfg = copy.deepcopy(NESE_A)
        change(cfg)
        with pytest.raises(ValueError):
            arch.build_spec(arch.read_config(cfg))


def test_a_borrowed_layer_may_be_named_in_turn():
    from paged_llm_amd.config.registry import lookup_architecture
    arch = lookup_architecture(NESE_A)
    cfg = copy.deepcopy(NESE_A)
    cfg["layers"].append(dict(copy.deepcopy(cfg["layers"][3]), weights_of=3))          # 6 -> 3 -> 0
    spec = arch.build_spec(arch.read_config(cfg))
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 0, 1, 2, 0] and len(spec.layers) == 3
    cfg["layers"][3]["weights_of"] = 6                                                 # 3 -> 6 -> 3: never ends
    with pytest.raises(ValueError):
        arch.build_spec(arch.read_config(cfg))


def test_rotary_frequencies_of_the_engine_are_the_plain_ones():
    """The engine's table builder (frequencies formed in double precision, the rescaling by wavelength) against the
    plain list, for the rescaling's three ranges."""
    from paged_llm_amd.parts.registry import BuildEnv, build as build_part
    from paged_llm_amd.parts.spec import PartSpec
    from paged_llm_amd.models.nesezen import _rotary
    for rot in ({"base": 1e4, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48}}, {"base": 33.0, "dims": 10},
                {"base": 5e5, "dims": 64, "scaling": {"factor": 8.0, "low": 2.0, "high": 8.0, "original": 512}}):
        spec = _rotary(rot, 64)
        env = BuildEnv(64, torch.float32, torch.device("cpu"), 32, shared={})
        part = build_part("position_encoding", PartSpec(**spec), env)
        want = torch.tensor(plain.rotary_frequencies(rot["base"], rot["dims"], rot.get("scaling")), dtype=torch.float32)
        assert torch.equal(part.inverse_frequencies(), want)
    kept = plain.rotary_frequencies(1e4, 16, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48})
    bare = plain.rotary_frequencies(1e4, 16, None)
    ranges = {("kept" if a == b else "slowed" if abs(a - b / 4.0) < 1e-12 * b else "blended") for a, b in zip(kept, bare)}
    assert ranges == {"kept", "slowed", "blended"}, "the test's constants reach all three ranges of wavelengths"


# --------------------------------------------------------------------------- the plain mechanisms against closed forms
def test_dynamic_tanh_is_elementwise():
    x = torch.randn(5, 7, dtype=torch.float64)
    w, b = torch.randn(7, dtype=torch.float64), torch.randn(7, dtype=torch.float64)
    y = plain.dynamic_tanh(x, torch.tensor(0.7, dtype=torch.float64), w, b)
    for t in range(5):
        for i in range(7):
            assert abs(float(y[t, i]) - (math.tanh(0.7 * float(x[t, i])) * float(w[i]) + float(b[i]))) < 1e-12


def test_rotation_turns_pairs_half_a_width_apart_and_leaves_the_rest():
    x = torch.randn(6, 2, 10, dtype=torch.float64)
    freqs = plain.rotary_frequencies(50.0, 6, None)
    y = plain.rotate(x, torch.arange(6), freqs, 6)
    for p in range(6):
        for i in range(3):
            a = float(torch.tensor(p, dtype=torch.float32) * torch.tensor(freqs[i], dtype=torch.float32))
            u, v = float(x[p, 1, i]), float(x[p, 1, i + 3])
            assert abs(float(y[p, 1, i]) - (u * math.cos(a) - v * math.sin(a))) < 1e-9
            assert abs(float(y[p, 1, i + 3]) - (v * math.cos(a) + u * math.sin(a))) < 1e-9
    assert torch.equal(y[..., 6:], x[..., 6:])


def test_windowed_attention_token_by_token():
    torch.manual_seed(1)
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "mask": {"size": 3}, "rot": {"base": 10.0, "dims": 4}, "scale": 0.7, "softcap": 2.0}
    T, W = 9, 12
    h = torch.randn(T, W, dtype=torch.float64)
    w = {"q": torch.randn(24, W, dtype=torch.float64), "k": torch.randn(12, W, dtype=torch.float64), "v": torch.randn(10, W, dtype=torch.float64),
         "o": torch.randn(W, 20, dtype=torch.float64)}
    got = plain.attention_mixer(h, w, m, torch.arange(T))
    freqs = plain.rotary_frequencies(10.0, 4, None)
    q = plain.rotate((h @ w["q"].T).view(T, 4, 6), torch.arange(T), freqs, 4)
    k = plain.rotate((h @ w["k"].T).view(T, 2, 6), torch.arange(T), freqs, 4)
    v = (h @ w["v"].T).view(T, 2, 5)
    for t in range(T):
        heads = []
        for head in range(4):
            g = head // 2
            js = [j for j in range(T) if 0 <= t - j < 3]
            s = torch.tensor([2.0 * math.tanh(float(q[t, head] @ k[j, g]) * 0.7 / 2.0) for j in js], dtype=torch.float64)
            p = torch.exp(s) / torch.exp(s).sum()
            heads.append(sum(p[n] * v[j, g] for n, j in enumerate(js)))
        assert torch.allclose(got[t], torch.cat(heads) @ w["o"].T, atol=1e-10)


def test_matrix_memory_against_the_sum_over_earlier_tokens():
    """Without the running maximum: S_t = sum_s exp(i_s + sum_(s < r <= t) f_r) k_s v_s^T, the same for n_t, and the
    output S_t^T q / max(|n_t . q|, 1) up to the 1e-6 (which stands beside exp(-m) in the stabilised form: compared where
    it does not matter)."""
    torch.manual_seed(2)
    m = {"heads": 2, "dim": 4, "vdim": 3, "gate_cap": 6.0}
    T, W = 11, 10
    h = torch.randn(T, W, dtype=torch.float64)
    w = {n: torch.randn(r, W, dtype=torch.float64) for n, r in (("q", 8), ("k", 8), ("v", 6), ("g", 6), ("i", 2), ("f", 2))}
    w.update({"i.b": torch.randn(2, dtype=torch.float64), "f.b": torch.randn(2, dtype=torch.float64) + 2.0, "norm": torch.randn(6, dtype=torch.float64),
              "o": torch.randn(W, 6, dtype=torch.float64)})
    got = plain.mlstm_mixer(h, w, m, 1e-5)
    q = (h @ w["q"].T).view(T, 2, 4) * 4 ** -0.5
    k, v = (h @ w["k"].T).view(T, 2, 4), (h @ w["v"].T).view(T, 2, 3)
    gi = 6.0 * torch.tanh((h @ w["i"].T + w["i.b"]) / 6.0)
    gf = torch.log(torch.sigmoid(6.0 * torch.tanh((h @ w["f"].T + w["f.b"]) / 6.0)))
    for t in range(T):
        heads = []
        for head in range(2):
            weight = [math.exp(float(gi[s, head]) + float(gf[s + 1:t + 1, head].sum())) for s in range(t + 1)]
            S = sum(wt * torch.outer(k[s, head], v[s, head]) for s, wt in enumerate(weight))
            n = sum(wt * k[s, head] for s, wt in enumerate(weight))
            m_t = max([float(gi[s, head]) + float(gf[s + 1:t + 1, head].sum()) for s in range(t + 1)] + [float(gf[:t + 1, head].sum())])
            o = (S.T @ q[t, head]) / (max(abs(float(n @ q[t, head])), 1.0) + 1e-6 * math.exp(m_t))
            heads.append(o / torch.sqrt((o * o).mean() + 1e-5))
        want = (torch.cat(heads) * w["norm"] * torch.sigmoid(h[t] @ w["g"].T)) @ w["o"].T
        assert torch.allclose(got[t], want, atol=1e-9, rtol=1e-9)


def test_latent_attention_against_keys_expanded_token_by_token():
    torch.manual_seed(3)
    m = {"heads": 3, "dim": 4, "vdim": 5, "kv_rank": 6, "q_rank": 7, "scale": 0.4}
    T, W = 8, 9
    h = torch.randn(T, W, dtype=torch.float64)
    w = {n: torch.randn(*s, dtype=torch.float64) for n, s in (("dq", (7, W)), ("dq.norm", (7,)), ("uq", (12, 7)), ("dkv", (6, W)), ("dkv.norm", (6,)),
                                                             ("uk", (12, 6)), ("uv", (15, 6)), ("g", (3, W)), ("o", (W, 15)))}
    got = plain.latent_attention_mixer(h, w, m, 1e-4, torch.arange(T))

    def normed(x, weight):
        return x / math.sqrt(float((x * x).mean()) + 1e-4) * weight
    for t in range(T):
        q = (w["uq"] @ normed(w["dq"] @ h[t], w["dq.norm"])).view(3, 4)
        cs = [normed(w["dkv"] @ h[j], w["dkv.norm"]) for j in range(t + 1)]
        heads = []
        for head in range(3):
            s = torch.stack([(q[head] @ (w["uk"] @ c).view(3, 4)[head]) * 0.4 for c in cs])
            p = torch.softmax(s, dim=0)
            out = sum(p[j] * (w["uv"] @ c).view(3, 5)[head] for j, c in enumerate(cs))
            heads.append(out * torch.sigmoid(w["g"][head] @ h[t]))
        assert torch.allclose(got[t], torch.cat(heads) @ w["o"].T, atol=1e-10)


def test_routed_experts_weigh_their_input():
    torch.manual_seed(4)
    W, ff = 6, 5
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": 4, "top": 2}, "shared": {"ff": 3}}
    w = {"router": torch.randn(4, W, dtype=torch.float64), "shared.sg": torch.randn(1, W, dtype=torch.float64)}
    for e in ["e0", "e1", "e2", "e3", "shared"]:
        f = 3 if e == "shared" else ff
        w.update({f"{e}.gate": torch.randn(f, W, dtype=torch.float64), f"{e}.up": torch.randn(f, W, dtype=torch.float64),
                  f"{e}.down": torch.randn(W, f, dtype=torch.float64)})
    h = torch.randn(5, W, dtype=torch.float64)
    got = plain.routed_feed_forward(h, w, mlp)
    for t in range(5):
        s = [1.0 / (1.0 + math.exp(-float(w["router"][e] @ h[t]))) for e in range(4)]
        chosen = sorted(range(4), key=lambda e: -s[e])[:2]
        want = torch.zeros(W, dtype=torch.float64)
        for e in chosen:
            x = s[e] * h[t]
            g, u = w[f"e{e}.gate"] @ x, w[f"e{e}.up"] @ x
            want += w[f"e{e}.down"] @ (g / (1.0 + torch.exp(-g)) * u)
        g, u = w["shared.gate"] @ h[t], w["shared.up"] @ h[t]
        want += (w["shared.down"] @ (g / (1.0 + torch.exp(-g)) * u)) / (1.0 + math.exp(-float(w["shared.sg"][0] @ h[t])))
        assert torch.allclose(got[t], want, atol=1e-10)
    ids, weights = plain.choose_experts(torch.zeros(1, W, dtype=torch.float64), w["router"], 2)
    assert ids.tolist() == [[0, 1]] and weights.tolist() == [[0.5, 0.5]], "equal scores: the lower index wins, the weights are not renormalised"


def test_the_whole_model_is_the_sum_of_its_branches():
    """One pass of the plain model over a configuration with every kind of layer against the same composition written
    out layer by layer with the mechanisms' functions."""
    import os
    import tempfile
    from paged_llm_amd.weights import write_random_model
    with tempfile.TemporaryDirectory() as d:
        folder = write_random_model(d, NESE_A, seed=1, dtype="float32", std=0.1, norm_jitter=True)
        cfg, w = plain.read_config(folder), plain.load_weights(folder)
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    seen = []
    logits = plain.forward(cfg, w, toks, layers_out=seen)
    assert len(seen) == 6 and logits.shape == (8, 300)
    x = w["embed"][torch.tensor(toks)]
    pos = torch.arange(8)
    for i, l in enumerate(cfg["layers"]):
        src = f"l{l.get('weights_of', i) if l.get('weights_of') is not None else i}"
        wm = {n[len(src) + 5:]: t for n, t in w.items() if n.startswith(src + ".mix.")}
        h = torch.tanh(w[src + ".norm1.alpha"] * x) * w[src + ".norm1"] + w[src + ".norm1.b"]
        x = x + {"attention": lambda: plain.attention_mixer(h, wm, l["mixer"], pos), "mlstm": lambda: plain.mlstm_mixer(h, wm, l["mixer"], 1e-5),
                 "latent_attention": lambda: plain.latent_attention_mixer(h, wm, l["mixer"], 1e-5, pos)}[l["type"]]()
        if l["mlp"] is not None:
            wf = {n[len(src) + 5:]: t for n, t in w.items() if n.startswith(src + ".mlp.")}
            h = torch.tanh(w[src + ".norm2.alpha"] * x) * w[src + ".norm2"] + w[src + ".norm2.b"]
            x = x + (plain.gated_feed_forward(h, wf) if l["mlp"]["kind"] == "dense" else plain.routed_feed_forward(h, wf, l["mlp"]))
        assert torch.allclose(seen[i], x, atol=1e-6)
    assert not torch.allclose(seen[0], seen[3]) and not torch.allclose(seen[1], seen[4])


def test_the_configuration_that_bench_measures_builds():
    """``bench.py --nesezen`` measures a configuration of its own making: it passes the registry and has the layers
    its description names."""
    import os
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if root not in sys.path:
        sys.path.insert(0, root)
    import bench
    from paged_llm_amd.config.registry import lookup_architecture
    for width in (1024, 2048):
        cfg = bench.nesezen_config(width, 32000)
        arch = lookup_architecture(cfg)
        spec = arch.build_spec(arch.read_config(cfg))
        assert len(spec.schedule) == len(spec.layers) == 12 and spec.hidden_size == width
        kinds = [l.parts["mixer"].kind for l in spec.layers]
        assert kinds.count("normed_attention") == 6 and kinds.count("mlstm") == 3 and kinds.count("latent_attention") == 3
        assert sum(l.parts["feed_forward"].kind == "routed_experts" for l in spec.layers) == 6

