"""Renadra in the engine against the plain implementation under tests/plain/: each mechanism alone, whole prompts,
token-by-token decoding, portions down to two tokens, unequal requests in one batch with pages and state slots used
again, keys far back, at page borders and on either side of a window's edge and of the kept first positions (with weights
made so that one score stands out), the first tokens of a sequence, long decoding, sizes of several kinds, and greedy
generation through ``LLMEngine``."""

import copy
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests.helpers import TraceBuilder
from tests.renadra_configs import ALONE, RENA_A, RENA_B, RENA_C, attention, dense, hgrn2, layer, left, model, parallel, right
from tests.plain import renadra_plain as plain

pytestmark = pytest.mark.gpu

CONFIGS = {"A": RENA_A, "B": RENA_B, "C": RENA_C, **ALONE}
TOL = {"float32": 3e-5, "bfloat16": 6e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def lively(tensors):
    """Lower bounds of the forget gates spread over (0, 1), forget gates and per-head score biases that differ from token
    to token and head to head, biases of the projections that are not small (weights of the usual size leave every gate near
    one half and every bias near nothing)."""
    gen = torch.Generator().manual_seed(5)
    for name in list(tensors):
        t = tensors[name]
        if name.endswith(".mix.lower"):
            tensors[name] = torch.sigmoid(torch.randn(t.shape, generator=gen) * 1.5).to(t.dtype)
        elif name.endswith(".mix.f"):
            tensors[name] = (t.float() * 6.0).to(t.dtype)
        elif name.endswith((".mix.f.b", ".left.pb")):
            tensors[name] = (torch.randn(t.shape, generator=gen) * 1.5).to(t.dtype)
        elif name.endswith((".q.b", ".k.b", ".v.b", ".o.b")):
            tensors[name] = (torch.randn(t.shape, generator=gen) * 0.3).to(t.dtype)


def write_folder(path, cfg, seed, stored, edit=None):
    from safetensors.torch import load_file, save_file
    from paged_llm_amd.weights import write_random_model
    folder = write_random_model(str(path), cfg, seed=seed, dtype=stored, std=cfg["width"] ** -0.5, norm_jitter=True)
    file = os.path.join(folder, "model.safetensors")
    tensors = load_file(file)
    lively(tensors)
    if edit is not None:
        edit(tensors)
    save_file({k: v.contiguous() for k, v in tensors.items()}, file)
    return folder


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, stored):
        if (name, stored) not in made:
            made[name, stored] = write_folder(tmp_path_factory.mktemp(f"renadra_{name}_{stored}"), CONFIGS[name],
                                              seed=29 + len(name), stored=stored)
        return made[name, stored]
    return get


_plain_cache: dict = {}


def plain_logits(folder, tokens):
    key = (folder, tuple(tokens))
    if key not in _plain_cache:
        _plain_cache[key] = plain.forward(plain.read_config(folder), plain.load_weights(folder), list(tokens)).numpy()
    return _plain_cache[key]


def session_for(folder, dtype, max_tokens, **kw):
    from paged_llm_amd.engine.replay import ReplaySession
    return ReplaySession(folder, dtype, max_tokens, None, **kw)


_noise_cache: dict = {}


def rounding_scale(folder, tokens):
    """Per position: how far the plain logits move (root mean square over four draws of ``helpers.worst``) when every
    product's rows and result carry the relative error of bfloat16 rounding."""
    key = (folder, tuple(tokens))
    if key not in _noise_cache:
        exact = plain_logits(folder, tokens)
        cfg, weights = plain.read_config(folder), plain.load_weights(folder)
        sq = np.zeros(len(tokens))
        for seed in range(4):
            with plain.rounding_noise(seed):
                moved = plain.forward(cfg, weights, list(tokens)).numpy()
            sq += (np.abs(moved - exact).max(axis=1) / np.abs(exact).max(axis=1)) ** 2
        _noise_cache[key] = np.sqrt(sq / 4)
    return _noise_cache[key]


_exact_cache: dict = {}


def float32_scale(folder, tokens):
    """Per position: how far the plain implementation in float32 is from itself in float64."""
    key = (folder, tuple(tokens))
    if key not in _exact_cache:
        exact = plain.forward(plain.read_config(folder), plain.load_weights(folder), list(tokens), dtype=torch.float64).numpy()
        _exact_cache[key] = np.abs(plain_logits(folder, tokens) - exact).max(axis=1) / np.abs(exact).max(axis=1)
    return _exact_cache[key]


def bound_at(folder, tokens, pos, dtype):
    """What a row may differ by: in float32 3e-5, or 5 times the plain implementation's own float32 error at that
    position if that is more; in bfloat16 4 times the position's rounding scale, at least 3e-2."""
    if dtype == "float32":
        return max(TOL[dtype], 5.0 * float(float32_scale(folder, tokens)[pos]))
    return max(3e-2, 4.0 * float(rounding_scale(folder, tokens)[pos]))


def check(got: dict, folder, reqs: dict, dtype, narrow=False):
    """Every row within its bound in float32.  In bfloat16: no row beyond twice its bound (four times for ``narrow`` models,
    whose few channels average little rounding away), at most one in fifty beyond it, and the median error below 2.5e-2."""
    want = {rid: plain_logits(folder, toks) for rid, toks in reqs.items()}
    ratios, errs = {}, []
    for (rid, pos), row in got.items():
        err = helpers.worst(row, want[rid][pos])
        errs.append(err)
        ratios[rid, pos] = err / bound_at(folder, reqs[rid], pos, dtype)
    worst_at = max(ratios, key=ratios.get)
    over = sum(1 for r in ratios.values() if r > 1.0)
    said = f"{worst_at}: {ratios[worst_at]:.3g} of its bound (median error {np.median(errs):.3g}), {over} of {len(ratios)} rows over"
    if dtype == "float32":
        assert ratios[worst_at] <= 1.0, said
    else:
        most, middle = (4.0, 5e-2) if narrow else (2.0, 2.5e-2)
        assert ratios[worst_at] <= most and over <= max(1, len(ratios) // 50) and np.median(errs) <= middle, said


def whole(reqs):
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        trace.step([(rid, toks, "all")], end=[rid])
    return trace


def prompt_then_single(rid, toks, cut, want="all"):
    trace = TraceBuilder().step([(rid, toks[:cut], want)], end=[rid] if cut == len(toks) else [])
    for i in range(cut, len(toks)):
        trace.step([(rid, toks[i:i + 1], "all")], end=[rid] if i == len(toks) - 1 else [])
    return trace


def stored_as(dtype):
    return "float32" if dtype == "float32" else "bfloat16"


# --------------------------------------------------------------------------- each mechanism alone, and whole models
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompts(folders, name, dtype):
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    reqs = {"p1": helpers.random_tokens(1, vocab, 1), "p5": helpers.random_tokens(5, vocab, 2), "p70": helpers.random_tokens(70, vocab, 3)}
    got = helpers.replay_in_process(session_for(folder, dtype, 128), whole(reqs))
    assert len(got) == 76
    check(got, folder, reqs, dtype, narrow=name == "B")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "left", "right", "attention", "hgrn2", "loop"])
def test_prompt_then_token_by_token(folders, name, dtype):
    """A prompt in one step and then single tokens: pages, the recurrences' state slots, the token before in its slot,
    windows whose edges pass among decoded tokens."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(75, CONFIGS[name]["vocab"], 7)
    session = session_for(folder, dtype, 128)
    check(helpers.replay_in_process(session, prompt_then_single("r", toks, 13)), folder, {"r": toks}, dtype, narrow=name == "B")
    assert any(key[0] != "prompt" for key in session.runner._graphs), "single-token steps are replayed from graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_token_by_token_from_the_first(folders, name, dtype):
    """No prompt step at all: the first token takes the bigram table's last row, the recurrences start from zeros, a window
    of one position sees the kept positions beside itself."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(12, CONFIGS[name]["vocab"], 8)
    check(helpers.replay_in_process(session_for(folder, dtype, 64), prompt_then_single("r", toks, 1)), folder, {"r": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16, 1, 17, 2, 31], [64, 5]])
def test_portions(folders, name, dtype, sizes):
    """Prompts cut into portions of several sizes, down to two tokens, cut in the middle of pages and windows and inside the
    kept first positions."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(97, CONFIGS[name]["vocab"], 9)
    trace, at, k = TraceBuilder(), 0, 0
    while at < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - at)
        trace.step([("r", toks[at:at + n], "all")], end=["r"] if at + n == len(toks) else [])
        at, k = at + n, k + 1
    check(helpers.replay_in_process(session_for(folder, dtype, 128), trace), folder, {"r": toks}, dtype, narrow=name == "B")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "hgrn2", "right"])
def test_long_portions_across_the_chunks_of_the_recurrences(folders, name, dtype):
    """Portions long enough that the recurrences run in chunks side by side (with a short sequence beside the long one), then
    a portion that continues from the state those left, then single tokens."""
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    reqs = {"long": helpers.random_tokens(437, vocab, 11), "short": helpers.random_tokens(9, vocab, 12)}
    trace = TraceBuilder().step([("long", reqs["long"][:301], "last"), ("short", reqs["short"][:7], "all")])
    trace.step([("long", reqs["long"][301:431], [0, 1, 63, 64, 65, 129]), ("short", reqs["short"][7:8], "all")])
    trace.step([("short", reqs["short"][8:], "all")], end=["short"])
    for i in range(431, 437):
        trace.step([("long", reqs["long"][i:i + 1], "all")], end=["long"] if i == 436 else [])
    check(helpers.replay_in_process(session_for(folder, dtype, 576), trace), folder, reqs, dtype, narrow=name == "B")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_logits_do_not_depend_on_the_cut(folders, name, dtype):
    """The same request whole, in portions and token by token: equal within rounding of the compute type."""
    folder = folders(name, stored_as(dtype))
    toks = helpers.random_tokens(60, CONFIGS[name]["vocab"], 10)
    a = helpers.replay_in_process(session_for(folder, dtype, 64), whole({"r": toks}))
    trace = TraceBuilder().step([("r", toks[:31], "all")]).step([("r", toks[31:33], "all")])
    for i in range(33, 60):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == 59 else [])
    b = helpers.replay_in_process(session_for(folder, dtype, 64), trace)
    if dtype == "float32":
        assert max(helpers.worst(b[k], a[k]) for k in a) <= 1e-5
    else:
        assert max(helpers.worst(b[k], a[k]) / bound_at(folder, toks, k[1], dtype) for k in a) <= 2.0


# --------------------------------------------------------------------------- batches, pages and slots used again
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    from tests.test_replay_gpu import mixed_trace
    folder = folders(name, stored_as(dtype))
    vocab = CONFIGS[name]["vocab"]
    lengths = [33, 1, 90, 17, 64, 5, 48, 2, 71]
    reqs = {f"q{i}": helpers.random_tokens(n, vocab, 40 + i) for i, n in enumerate(lengths)}
    trace, peak = mixed_trace(reqs, max_live=3, seed=3)
    session = session_for(folder, dtype, peak, max_requests=3)
    got = helpers.replay_in_process(session, trace)
    assert len(got) == sum(lengths)
    check(got, folder, reqs, dtype, narrow=name == "B")
    session.manager.check_invariants()
    assert session.manager.slots.num_free == session.manager.slots.num_slots == 3
    assert all(session.manager.num_free_pages(g) == session.manager.num_pages(g) for g in session.manager.groups)
    kinds = {"prompt" if key[0] == "prompt" else "decode" for key in session.runner._graphs}
    assert kinds == {"prompt", "decode"}, "steps of both kinds were replayed from graphs"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_that_held_another_request_starts_from_zero(folders, dtype):
    """One state slot, a page pool of one request: the second request gets the slot (the first one's states and last token in
    it) and the pages the first one left full."""
    folder = folders("A", stored_as(dtype))
    reqs = {"first": helpers.random_tokens(50, RENA_A["vocab"], 60), "second": helpers.random_tokens(44, RENA_A["vocab"], 61)}
    trace = TraceBuilder()
    for rid, toks in reqs.items():
        trace.step([(rid, toks[:20], "all")])
        trace.step([(rid, toks[20:22], "all")])
        for i in range(22, len(toks)):
            trace.step([(rid, toks[i:i + 1], "all")], end=[rid] if i == len(toks) - 1 else [])
    session = session_for(folder, dtype, 64, max_requests=1)
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """Two hundred single tokens behind a short prompt: the windows pass over decoded tokens several times, pages of the
    windowed groups go back to the pool on the way while the pages of the kept positions stay, the states move two hundred
    times."""
    folder = folders("A", stored_as(dtype))
    toks = helpers.random_tokens(215, RENA_A["vocab"], 70)
    session = session_for(folder, dtype, 256)
    check(helpers.replay_in_process(session, prompt_then_single("r", toks, 15)), folder, {"r": toks}, dtype)


# --------------------------------------------------------------------------- where random weights would hide a fault
def aim_tokens(cfg, tensors, prefix, key_token, query_token, strength):
    """Make ``key_token``'s embedding a large multiple of unit vector a and ``query_token``'s of unit vector b (the bigram
    table is emptied, so a token's stream row is its embedding), and let column a of head 0's key rows and column b of head
    0's query rows (tensors under ``prefix``) carry one vector of squared length ``strength`` on the dimensions that are not
    rotated: wherever that key is visible to that query their score towers over all others."""
    layer0 = cfg["layers"][0]["mixer"]
    m = layer0["left"] if "left" in layer0 else layer0
    d, r, width = int(m["dim"]), int(m["rot"]["dims"]), cfg["width"]
    a, b = 1, 2
    gen = torch.Generator().manual_seed(77)
    target = torch.zeros(d, dtype=torch.float64)
    target[r:] = torch.randn(d - r, generator=gen, dtype=torch.float64)
    target *= (strength / float(target @ target)) ** 0.5
    tensors["bigram"] = torch.zeros_like(tensors["bigram"])
    norm_w = tensors["l0.norm1"].to(torch.float64)
    for token, matrix, col in ((key_token, prefix + "k", a), (query_token, prefix + "q", b)):
        e = torch.zeros(width, dtype=torch.float64)
        e[col] = 2.0
        tensors["embed"][token] = (e / cfg["embedding"]["scale"]).to(tensors["embed"].dtype)
        w = tensors[matrix].to(torch.float64)
        w[:d, col] = target / (width ** 0.5 * float(norm_w[col]))        # the normed row is sqrt(width) * w[col] along that unit vector
        tensors[matrix] = w.to(tensors[matrix].dtype)
        tensors[matrix + ".b"][:d] = 0


def _edge_case(tmp_path, dtype, kind, size, key_pos, seed, keep_first=0):
    """A one-layer model whose window has ``size``, a key at ``key_pos`` and queries aimed at it on both sides of the place
    where it leaves sight.  Returns (folder, tokens, last position that sees it, first that does not)."""
    if kind == "left":
        mixer = parallel(left(heads=2, kv_heads=1, dim=32, size=size, keep_first=keep_first, rot_dims=4, base=100.0, scale=0.5, softcap=50.0, scaling=None),
                         right(heads=1, dim=8, vdim=8), left_scale=1.0, right_scale=0.3)
        cfg, prefix = model(128, 120, [layer("parallel", mixer)], eps=1e-6), "l0.mix.left."
    else:
        mixer = attention(heads=2, kv_heads=1, dim=32, vdim=16, size=size, rot_dims=4, base=100.0, scale=0.5)
        cfg, prefix = model(128, 120, [layer("attention", mixer)], eps=1e-6), "l0.mix."
    edge_in = key_pos + size - 1
    n = edge_in + 6
    toks = [5 + t % 100 for t in helpers.random_tokens(n, 100, seed)]
    toks[key_pos] = 4                                       # the key's token stands nowhere else
    for pos in (edge_in - 1, edge_in, edge_in + 1, edge_in + 2):
        toks[pos] = 3                                       # ... and the aimed query's token only here

    def edit(t):
        aim_tokens(cfg, t, prefix, 4, 3, 64.0)
        if kind == "left":
            t["l0.mix.left.pb"] = torch.full_like(t["l0.mix.left.pb"], -16.0)          # other keys weigh little, the aimed one nearly one
    folder = write_folder(tmp_path, cfg, seed=seed, stored=stored_as(dtype), edit=edit)
    return folder, toks, edge_in, edge_in + 1


def _mask_of(cfg):
    m = cfg["layers"][0]["mixer"]
    return (m["left"] if "left" in m else m)["mask"]


def _assert_edge_shows(folder, toks, edge_in, edge_out, dtype, field="size"):
    """The plain implementation with a window (or a number of kept positions) one larger or smaller differs far beyond the
    bound at the edge."""
    want = plain_logits(folder, toks)
    for off_by in (-1, 1):
        other = plain.read_config(folder)
        _mask_of(other)[field] += off_by
        moved = plain.forward(other, plain.load_weights(folder), toks).numpy()
        pos = edge_in if off_by < 0 else edge_out
        assert helpers.worst(moved[pos], want[pos]) > 5 * bound_at(folder, toks, pos, dtype), "the aimed key does not show at the edge"
    return want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["left", "attention"])
@pytest.mark.parametrize("size,key_pos", [(9, 20), (130, 3), (64, 63), (16, 16), (33, 15)])
def test_edges_of_windows_in_prompts_and_in_decoding(tmp_path, kind, size, key_pos, dtype):
    """One key that the queries near the edge score far above all others: the last position that sees it and the first
    that does not are compared whole, with the edge among decoded tokens, with everything behind the key decoded and
    with the edge at the start of a portion of two tokens.  Small windows, windows of more than two pages (the key far
    back, over page borders) and windows of whole pages with the key on a page's first or last place; under a softmax and
    under sigmoid weights."""
    folder, toks, edge_in, edge_out = _edge_case(tmp_path, dtype, kind, size, key_pos, seed=31)
    want = _assert_edge_shows(folder, toks, edge_in, edge_out, dtype)
    n = len(toks)
    traces = {"whole": prompt_then_single("r", toks, n), "edge decoded": prompt_then_single("r", toks, edge_in - 3),
              "all decoded": prompt_then_single("r", toks, key_pos + 1),
              "edge starts a portion": TraceBuilder().step([("r", toks[:edge_in], "all")]).step([("r", toks[edge_in:edge_in + 2], "all")])
              .step([("r", toks[edge_in + 2:], "all")], end=["r"])}
    for label, trace in traces.items():
        got = helpers.replay_in_process(session_for(folder, dtype, -(-n // 64) * 64), trace)
        for pos in (edge_in - 1, edge_in, edge_out, edge_out + 1):
            err = helpers.worst(got["r", pos], want[pos])
            assert err <= 2.0 * bound_at(folder, toks, pos, dtype), f"{label}, position {pos}: {err:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("keep,size", [(3, 9), (16, 16), (21, 40), (1, 1)])
def test_the_last_kept_position_and_the_first_that_is_not(tmp_path, keep, size, dtype):
    """The aimed key stands on the last kept position, then on the first position that is not kept, far behind the window:
    queries hundreds of tokens later see the one and not the other, in prompts, in portions and among decoded tokens, while the
    pages between the kept ones and the window have gone back to the pool."""
    for key_pos, seen in ((keep - 1, True), (keep, False)):
        folder, toks, _, _ = _edge_case(tmp_path / f"k{key_pos}", dtype, "left", size, key_pos, seed=41, keep_first=keep)
        n = key_pos + size + 150
        toks = (toks + [5 + t % 100 for t in helpers.random_tokens(n, 100, 43)])[:n]
        toks = [5 if t == 3 else t for t in toks]             # the aimed query stands at two late positions only
        toks[key_pos] = 4
        for pos in (n - 40, n - 3):
            toks[pos] = 3
        want = plain_logits(folder, toks)
        other = plain.read_config(folder)
        _mask_of(other)["keep_first"] += -1 if seen else 1
        moved = plain.forward(other, plain.load_weights(folder), toks).numpy()
        for pos in (n - 40, n - 3):
            assert helpers.worst(moved[pos], want[pos]) > 5 * bound_at(folder, toks, pos, dtype), "the kept key does not show"
        cut = n - 20
        traces = {"whole": prompt_then_single("r", toks, n), "decoded": prompt_then_single("r", toks, cut, want=[n - 40]),
                  "portions": TraceBuilder().step([("r", toks[:keep + 1], [])]).step([("r", toks[keep + 1:n - 41], [])])
                  .step([("r", toks[n - 41:n - 39], "all")]).step([("r", toks[n - 39:], "all")], end=["r"])}
        for label, trace in traces.items():
            session = session_for(folder, dtype, -(-n // 64) * 64)
            got = helpers.replay_in_process(session, trace)
            for pos in (n - 40, n - 3):
                err = helpers.worst(got["r", pos], want[pos])
                assert err <= 2.0 * bound_at(folder, toks, pos, dtype), f"{label}, key at {key_pos}, position {pos}: {err:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["left", "attention"])
def test_a_key_far_back_among_hundreds(tmp_path, kind, dtype):
    """A window of 400 positions, the aimed key 390 tokens back among as many others, over two dozen page borders,
    through portions and decoded tokens."""
    folder, toks, edge_in, edge_out = _edge_case(tmp_path, dtype, kind, 400, 7, seed=37)
    want = _assert_edge_shows(folder, toks, edge_in, edge_out, dtype)
    trace, at = TraceBuilder(), 0
    for n in (17, 2, 64, 100, 3, 96, 60):
        trace.step([("r", toks[at:at + n], "last")])
        at += n
    for i in range(at, len(toks)):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == len(toks) - 1 else [])
    got = helpers.replay_in_process(session_for(folder, dtype, 448), trace)
    check(got, folder, {"r": toks}, dtype)
    assert ("r", edge_in) in got and ("r", edge_out) in got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["hgrn2", "right"])
def test_a_state_that_keeps_an_early_token(tmp_path, name, dtype):
    """Decays near one (forget gates held open by a large bias and a high lower bound; a decay of 0.999): what the first
    tokens wrote still carries the output 300 tokens later, through chunks, portions and decoded tokens.  The plain
    implementation started behind those tokens differs beyond the bound at the end."""
    cfg = copy.deepcopy(ALONE[name])
    if name == "right":
        cfg["layers"][0]["mixer"]["right"]["decay"] = [0.999, 0.9995]

    def edit(tensors):
        if name == "hgrn2":
            tensors["l0.mix.f.b"] = torch.full_like(tensors["l0.mix.f.b"], 5.0)
            tensors["l0.mix.f"] = (tensors["l0.mix.f"].float() * 0.05).to(tensors["l0.mix.f"].dtype)
            tensors["l0.mix.lower"] = torch.full_like(tensors["l0.mix.lower"], 0.9)
        tensors["bigram"] = (tensors["bigram"].float() * 0.1).to(tensors["bigram"].dtype)
    folder = write_folder(tmp_path, cfg, seed=47, stored=stored_as(dtype), edit=edit)
    toks = [5 + t % 100 for t in helpers.random_tokens(320, 100, 19)]
    want = plain_logits(folder, toks)
    c, w = plain.read_config(folder), plain.load_weights(folder)
    layer0, x = c["layers"][0], None
    # the stream rows are the embedding's, so the mixer started 40 tokens late shows what those 40 tokens still carry
    emb = plain.embedding(toks, w["embed"].float(), w["bigram"].float(), c["embedding"]["scale"], c["embedding"]["bigram"])
    h = plain.rms_norm(emb, w["l0.norm1"].float(), c["norm"]["eps"])
    wm = {k[len("l0.mix."):]: t.float() for k, t in w.items() if k.startswith("l0.mix.")}
    if name == "hgrn2":
        full, late = plain.hgrn2(h, wm, layer0["mixer"], c["norm"]["eps"]), plain.hgrn2(h[40:], wm, layer0["mixer"], c["norm"]["eps"])
    else:
        wr = {k[len("right."):]: t for k, t in wm.items() if k.startswith("right.")}
        full = plain.lightning_attention(h, wr, layer0["mixer"]["right"], c["norm"]["eps"])
        late = plain.lightning_attention(h[40:], wr, layer0["mixer"]["right"], c["norm"]["eps"])
    assert float((full[-1] - late[-1]).abs().max()) > 0.05 * float(full[-1].abs().max()), "the early tokens do not show at the end"
    trace, at = TraceBuilder(), 0
    for n in (3, 2, 140, 100, 2, 50):
        trace.step([("r", toks[at:at + n], "last")])
        at += n
    for i in range(at, len(toks)):
        trace.step([("r", toks[i:i + 1], "all")], end=["r"] if i == len(toks) - 1 else [])
    check(helpers.replay_in_process(session_for(folder, dtype, 320), trace), folder, {"r": toks}, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_token_before_a_portion_decides_its_first_row(tmp_path, dtype):
    """A bigram table as large as the token table (its rows weigh as much as the tokens'): a portion's first token takes the row
    of the pair with the token the step before ended on, for portions of two tokens, single tokens and a second request beside
    the first whose slot held another request's last token."""
    cfg = model(64, 120, [layer("hgrn2", hgrn2(heads=1, dim=8, vdim=8), dense(32))], bigram=(97, 11, 13))
    folder = write_folder(tmp_path, cfg, seed=3, stored=stored_as(dtype), edit=lambda t: t.update({"bigram": (t["bigram"].float() * 3.0).to(t["bigram"].dtype)}))
    reqs = {"a": helpers.random_tokens(23, 120, 1), "b": helpers.random_tokens(9, 120, 2), "c": helpers.random_tokens(6, 120, 3)}
    moved = plain.read_config(folder)
    moved["embedding"]["bigram"]["mul_prev"] += 1
    assert helpers.worst(plain.forward(moved, plain.load_weights(folder), reqs["a"]).numpy()[5], plain_logits(folder, reqs["a"])[5]) > 0.1
    a, b, c = reqs["a"], reqs["b"], reqs["c"]
    trace = TraceBuilder().step([("a", a[:2], "all"), ("b", b[:1], "all")]).step([("a", a[2:4], "all"), ("b", b[1:2], "all")])
    trace.step([("a", a[4:5], "all"), ("b", b[2:], "all")], end=["b"]).step([("a", a[5:16], "all"), ("c", c[:3], "all")])
    trace.step([("c", c[3:5], "all"), ("a", a[16:17], "all")]).step([("a", a[17:], "all"), ("c", c[5:], "all")], end=["a", "c"])
    session = session_for(folder, dtype, 64, max_requests=2)
    check(helpers.replay_in_process(session, trace), folder, reqs, dtype)


def random_config(seed):
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(0, len(xs)))]
    width = int(pick(40, 64, 72, 128))
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        kind = pick("parallel", "attention", "hgrn2")
        kv = int(pick(1, 2, 3))
        dim = int(pick(8, 16, 20, 48))
        rot = int(pick(0, 2, dim // 2 * 2, dim))
        size = int(pick(1, 7, 16, 32, 50, 500))
        if kind == "attention":
            m = attention(heads=kv * int(pick(1, 2, 4)), kv_heads=kv, dim=dim, vdim=int(pick(8, 16, 24, 72)), size=size, rot_dims=rot,
                          base=float(pick(10.0, 1e4, 5e5)), scale=float(pick(0.1, 0.3)))
        elif kind == "hgrn2":
            m = hgrn2(heads=int(pick(1, 2, 5)), dim=int(pick(4, 16, 33, 96)), vdim=int(pick(8, 31, 63, 64, 100)))
        else:
            heads_r = int(pick(1, 2, 5))
            m = parallel(left(heads=kv * int(pick(1, 2, 4)), kv_heads=kv, dim=dim, size=size, keep_first=int(pick(0, 1, 5, 16, 40)), rot_dims=rot,
                              base=float(pick(10.0, 1e4, 5e5)), scale=float(pick(0.1, 0.3)), softcap=float(pick(0.0, 3.0, 40.0)),
                              scaling=pick(None, {"factor": 8.0, "original": 32, "fast": 16.0, "slow": 2.0}, {"factor": 2.0, "original": 96, "fast": 4.0, "slow": 1.0})),
                         right(heads=heads_r, dim=int(pick(4, 16, 33, 96)), vdim=int(pick(8, 31, 64, 100)), decay=[float(rng.uniform(0.3, 1.0)) for _ in range(heads_r)]),
                         left_scale=float(pick(0.5, 1.0, 1.7)), right_scale=float(pick(0.25, 1.0)))
        layers.append(layer(kind, m, dense(int(pick(24, 100))) if rng.random() < 0.7 else None))
    n, loop = len(layers), None
    if rng.random() < 0.6:
        start = int(rng.integers(0, n))
        loop = (start, int(rng.integers(start + 1, n + 1)), int(rng.integers(1, 4)))
    return model(width, int(pick(50, 200, 333)), layers, eps=float(pick(1e-6, 1e-5, 1e-2)), scale=float(pick(0.3, 1.0, 2.0)),
                 bigram=(int(pick(1, 13, 257, 4099)), int(pick(1, 31, 1000003)), int(pick(1, 7, 65537))), loop=loop)


@pytest.mark.parametrize("seed", range(10))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Sizes, constants, options and layer orders drawn at random, in float32: a prompt, a portion of two tokens, single
    tokens, with a second request beside the first."""
    cfg = random_config(2000 + seed)
    folder = write_folder(tmp_path, cfg, seed=seed, stored="float32")
    reqs = {"a": helpers.random_tokens(83, cfg["vocab"], seed), "b": helpers.random_tokens(21, cfg["vocab"], 100 + seed)}
    trace = TraceBuilder().step([("a", reqs["a"][:49], "all")]).step([("a", reqs["a"][49:51], "all"), ("b", reqs["b"][:18], "all")])
    for i in range(51, 83):
        k = i - 51 + 18
        trace.step([("a", reqs["a"][i:i + 1], "all")] + ([("b", reqs["b"][k:k + 1], "all")] if k < 21 else []),
                   end=(["a"] if i == 82 else []) + (["b"] if k == 20 else []))
    got = helpers.replay_in_process(session_for(folder, "float32", 192), trace)
    assert len(got) == 104
    check(got, folder, reqs, "float32")


# --------------------------------------------------------------------------- the engine's own entry point
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_engine(folders, name):
    """``LLMEngine.generate`` with portions of 16 tokens, three requests at a time for five prompts (state slots and
    pages are used again): every row the engine sampled from is within the bound of the plain logits along its own
    tokens, and in float32 the tokens are the plain implementation's greedy choice."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    vocab = CONFIGS[name]["vocab"]
    prompts = [helpers.random_tokens(n, vocab, 70 + n) for n in (3, 41, 18, 1, 29)]
    for dtype in ("float32", "bfloat16"):
        folder = folders(name, stored_as(dtype))
        engine = LLMEngine(folder, EngineConfig(dtype=dtype, num_gpu_blocks=24, block_size=16, max_num_batched_tokens=16,
                                                max_num_seqs=3, max_model_len=128))
        rows = {}

        def keep(requests, logits):
            for r, row in zip(requests, logits.float().cpu()):
                rows[r.id, len(r.tokens) - 1] = row.numpy()
        engine.on_logits = keep
        outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
        assert engine.cache_manager.slots.num_free == 3
        for p, o in zip(prompts, outs):
            assert len(o.token_ids) == 12
            want = plain_logits(folder, p + o.token_ids)
            for i, token in enumerate(o.token_ids):
                pos = len(p) + i - 1
                err = helpers.worst(rows[o.seq_id, pos], want[pos])
                assert err <= 2.0 * bound_at(folder, p + o.token_ids, pos, dtype) and int(rows[o.seq_id, pos].argmax()) == token, (dtype, pos, err)
                if dtype == "float32":
                    top2 = np.sort(want[pos])[-2:]
                    if top2[1] - top2[0] > 1e-3 * np.abs(want[pos]).max():
                        assert token == int(want[pos].argmax()), (pos, token)


def test_preempted_requests_start_again_from_an_empty_state(folders):
    """A page pool too small for three requests at once: the scheduler preempts the request admitted last (pages and state
    slot given back, its tokens kept) and computes it again later as a longer prompt, from position 0: from zero states and
    with no token before, in whatever slot it gets.  Float32: the tokens are the plain implementation's greedy choice all the
    same."""
    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
    folder = folders("A", "float32")
    vocab = RENA_A["vocab"]
    prompts = [helpers.random_tokens(n, vocab, 400 + n) for n in (30, 22, 27)]
    engine = LLMEngine(folder, EngineConfig(dtype="float32", num_gpu_blocks=7, block_size=16, max_num_batched_tokens=32,
                                            max_num_seqs=3, max_model_len=128))
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True))
    assert engine.stats.num_preemptions > 0 and sum(o.num_preemptions for o in outs) > 0
    assert engine.cache_manager.slots.num_free == 3
    for p, o in zip(prompts, outs):
        assert len(o.token_ids) == 40
        want = plain_logits(folder, p + o.token_ids)
        for i, token in enumerate(o.token_ids):
            row = want[len(p) + i - 1]
            top2 = np.sort(row)[-2:]
            if top2[1] - top2[0] > 1e-3 * np.abs(row).max():
                assert token == int(row.argmax()), (len(p), i)


def test_the_replay_program_and_the_command_line(folders, tmp_path):
    folder = folders("B", "float32")
    toks = helpers.random_tokens(30, RENA_B["vocab"], 5)
    trace = TraceBuilder().step([("r", toks[:20], "last")]).step([("r", toks[20:], "all")], end=["r"])
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                          input=trace.jsonl(), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1"]
    got = helpers.read_replay_output(str(out), trace, RENA_B["vocab"])
    check(got, folder, {"r": toks}, "float32")
    gen = subprocess.run([sys.executable, os.path.join(ROOT, "examples", "generate.py"), "--model", folder, "--dtype", "float32",
                          "--prompt-ids", ",".join(str(t) for t in toks[:9]), "--prompt-ids", "9", "--max-tokens", "5", "--num-gpu-blocks", "16",
                          "--max-model-len", "64", "--ignore-eos"], capture_output=True, text=True, timeout=600)
    assert gen.returncode == 0, gen.stderr[-2000:]
