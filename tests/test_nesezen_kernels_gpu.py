"""The kernels that came with Nesezen, each against a plain PyTorch float32 (or float64) version of the same operation:
the norm without statistics with and without the residual sum and with the experts' sum formed inside, the gates of the
matrix memory and the recurrence with a normaliser, what follows that recurrence, the router with sigmoid scores and
outputs that ride along, experts whose weights stand on their inputs, the sum with a shared feed-forward, the latent's
preparation from float sums with a latent of the queries, and the attention preparation without the division."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(t):
    return t.to("cuda")


def randn(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


@pytest.mark.parametrize("hidden", [50, 64, 320, 2048, 4100])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_dynamic_tanh_with_and_without_the_sum(hidden, out_dtype):
    from paged_llm_amd.csrc import ops
    x, d = randn(7, hidden, seed=1) * 2.0, randn(7, hidden, seed=2)
    w, b = randn(hidden, seed=3), randn(hidden, seed=4)
    tol = 1e-6 if out_dtype == torch.float32 else 1e-2
    got = ops.dynamic_tanh(dev(x), 0.7, dev(w), dev(b), None, None, out_dtype)
    assert torch.allclose(got.float().cpu(), torch.tanh(0.7 * x) * w + b, atol=tol, rtol=tol)
    idx = torch.tensor([5, 0, 5], dtype=torch.int32)
    got = ops.dynamic_tanh(dev(x), 0.7, dev(w), dev(b), None, dev(idx), out_dtype)
    assert torch.allclose(got.float().cpu(), (torch.tanh(0.7 * x) * w + b)[idx.long()], atol=tol, rtol=tol)
    stream = dev(x.clone())
    got = ops.dynamic_tanh(stream, 1.3, dev(w), dev(b), dev(d), None, out_dtype)
    assert torch.equal(stream.cpu(), x + d), "the residual sum is one float addition"
    assert torch.allclose(got.float().cpu(), torch.tanh(1.3 * (x + d)) * w + b, atol=tol, rtol=tol)
    stream = dev(x.clone())
    ops.stream_add(stream, dev(d))
    assert torch.equal(stream.cpu(), x + d)


@pytest.mark.parametrize("cap", [0.0, 3.0, 15.0])
def test_gates_of_the_matrix_memory(cap):
    """Three sequences (one that starts, one that goes on from a stored maximum, one without tokens), lengths over the
    scan's blocks of 64 tokens, against the recurrence token by token."""
    from paged_llm_amd.csrc import ops
    H = 3
    lens, starts = [150, 70, 0, 1], [0, 9, 4, 0]
    T = sum(lens)
    raw = randn(T, 2 * H + 5, seed=5) * 6.0
    bi, bf = randn(H, seed=6), randn(H, seed=7) + 1.0
    state = randn(5, 40, seed=8)
    slots = torch.tensor([3, 1, 0, 2], dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    st = dev(state.clone())
    rows = dev(raw)
    decay, take, m = ops.mlstm_gates(rows[:, 2:2 + H], rows[:, 2 + H:2 + 2 * H], dev(bi), dev(bf), cap, st, 30, dev(slots),
                                     dev(torch.tensor(starts, dtype=torch.int32)), dev(cu), 4)
    want_state = state.clone().double()
    for s, (n, start) in enumerate(zip(lens, starts)):
        if n == 0:
            continue
        for h in range(H):
            mm = float(state[slots[s], 30 + h]) if start > 0 else 0.0
            for t in range(int(cu[s]), int(cu[s]) + n):
                gi, gf = float(raw[t, 2 + h]) + float(bi[h]), float(raw[t, 2 + H + h]) + float(bf[h])
                if cap > 0:
                    gi, gf = cap * math.tanh(gi / cap), cap * math.tanh(gf / cap)
                gf = min(gf, 0.0) - math.log1p(math.exp(-abs(gf)))
                new = max(gf + mm, gi)
                assert abs(float(m[t, h]) - new) <= 1e-5 * max(1.0, abs(new))
                assert abs(float(decay[t, h]) - math.exp(gf + mm - new)) <= 2e-5 and abs(float(take[t, h]) - math.exp(gi - new)) <= 2e-5
                mm = new
            want_state[slots[s], 30 + h] = mm
    assert torch.allclose(st.cpu().double(), want_state, atol=1e-4), "the last maximum of every sequence with tokens is left in its slot, nothing else moves"


@pytest.mark.parametrize("N,P", [(16, 24), (70, 66), (128, 64)])
@pytest.mark.parametrize("long", [False, True])
def test_recurrence_with_a_normaliser(N, P, long):
    """S and, as its last column, n under given decays and input factors: single tokens and short portions token by token,
    long portions in chunks."""
    from paged_llm_amd.csrc import ops
    H = 2
    lens, starts = ([200, 3], [0, 5]) if long else ([5, 1, 17], [0, 3, 0])
    T = sum(lens)
    q, k, v = randn(T, H, N, seed=1), randn(T, H, N, seed=2), randn(T, H, P, seed=3)
    decay, take = torch.rand(T, H, generator=torch.Generator().manual_seed(4)) * 0.5 + 0.5, torch.rand(T, H, generator=torch.Generator().manual_seed(5))
    state = randn(4, H * N * (P + 1) + 7, seed=6)
    slots = torch.tensor([2, 0, 3][:len(lens)], dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    st = dev(state.clone())
    y = ops.linear_recurrence(dev(q), dev(k), dev(v), dev(decay), st, 0, dev(slots), dev(torch.tensor(starts, dtype=torch.int32)), dev(cu),
                              len(lens), vscale=dev(take), max_q_len=max(lens), normaliser=True).cpu()
    for s, (n, start) in enumerate(zip(lens, starts)):
        S = state[slots[s], :H * N * (P + 1)].view(H, N, P + 1).double() if start > 0 else torch.zeros(H, N, P + 1, dtype=torch.float64)
        for t in range(int(cu[s]), int(cu[s]) + n):
            v1 = torch.cat([v[t].double(), torch.ones(H, 1, dtype=torch.float64)], dim=1)
            S = decay[t].double()[:, None, None] * S + take[t].double()[:, None, None] * (k[t].double()[:, :, None] * v1[:, None, :])
            want = torch.einsum("hnp,hn->hp", S, q[t].double()).reshape(-1)
            assert torch.allclose(y[t].double(), want, atol=2e-4, rtol=2e-4), (s, t)
        assert torch.allclose(st[slots[s], :H * N * (P + 1)].cpu().double(), S.reshape(-1), atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("P", [24, 66, 300])
def test_what_follows_the_matrix_memory(P, out_dtype):
    from paged_llm_amd.csrc import ops
    T, H = 9, 3
    y = randn(T, H * (P + 1), seed=1)
    y.view(T, H, P + 1)[0, 0, P] = 1e-4                   # a normaliser below exp(-m): the maximum takes over
    m = randn(T, H, seed=2) * 3.0
    rows = randn(T, H * P + 11, seed=3)
    w = randn(H * P, seed=4)
    got = ops.mlstm_output(dev(y), dev(m), dev(rows)[:, 4:4 + H * P], dev(w), H, P, 0.25, 1e-5, out_dtype).float().cpu()
    yy = y.view(T, H, P + 1).double()
    den = torch.maximum((yy[:, :, P] * 0.25).abs(), torch.exp(-m.double())) + 1e-6
    o = yy[:, :, :P] * 0.25 / den[:, :, None]
    o = o / torch.sqrt((o * o).mean(dim=2, keepdim=True) + 1e-5)
    want = o.reshape(T, H * P) * w.double() * torch.sigmoid(rows[:, 4:4 + H * P].double())
    tol = 2e-5 if out_dtype == torch.float32 else 1e-2
    assert torch.allclose(got.double(), want, atol=tol, rtol=tol)


@pytest.mark.parametrize("tokens", [1, 5, 200, 700])
@pytest.mark.parametrize("n,top,extra", [(8, 1, 1), (6, 2, 0), (5, 5, 1), (40, 7, 3)])
def test_router_with_sigmoid_scores_and_outputs_that_ride_along(tokens, n, top, extra):
    from paged_llm_amd.csrc import ops
    W = 96
    h = randn(tokens, W, seed=1)
    router = randn(n + extra, W, seed=2) * 0.3
    out = ops.moe_route(dev(h), dev(router), None, 1, 1, top, "sigmoid", extra=extra)
    ids, weights = out[0].cpu(), out[1].cpu()
    z = h.double() @ router.double().T
    s = torch.sigmoid(z[:, :n])
    order = torch.sort(s, dim=1, descending=True, stable=True).indices[:, :top]
    close = (torch.sort(s, dim=1, descending=True).values[:, :top + 1].diff(dim=1).abs().min(dim=1).values < 1e-6) if top < n else torch.zeros(tokens, dtype=torch.bool)
    assert torch.equal(ids[~close].long(), order[~close])
    assert torch.allclose(weights[~close].double(), torch.gather(s, 1, order)[~close], atol=1e-5)
    if extra:
        assert torch.allclose(out[2].cpu().double(), z[:, n:], atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens,experts,top", [(3, 4, 2), (300, 4, 1), (1200, 3, 2)])
def test_experts_with_weights_on_their_inputs_and_a_shared_one(tokens, experts, top, dtype):
    """All three tile sizes of the experts' products with a factor per pair on the input row, then the sum with a shared
    feed-forward's rows and a gate per token, by the sum's own kernel and by the kernel that also adds and norms."""
    from paged_llm_amd.csrc import ops
    W, ff = 64, 48
    h = (randn(tokens, W, seed=1) * 0.5).to(dtype)
    wgu = (randn(experts, 2 * ff, W, seed=2) * 0.2).to(dtype)
    wd = (randn(experts, W, ff, seed=3) * 0.2).to(dtype)
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand(tokens, top, generator=g) * 0.8 + 0.1
    shared, gate = randn(tokens, W, seed=5), randn(tokens, 3, seed=6)
    rows = ops.moe_tile_rows(ids.numel(), experts, dtype, W, ff, W)
    sorted_pair, row_of_pair, tiles = ops.moe_align(dev(ids), experts, rows)
    act = ops.moe_expert_gemm(dev(h), dev(wgu), tiles, sorted_pair, top, True, "silu", tile_rows=rows, pair_scale=dev(weights))
    out = ops.moe_expert_gemm(act, dev(wd), tiles, sorted_pair, top, False, tile_rows=rows)
    gate_dev = dev(gate)[:, 1:2]
    y = ops.moe_combine(out, dev(h), row_of_pair, dev(weights), True, dev(shared), gate_dev).cpu().double()
    want = torch.zeros(tokens, W, dtype=torch.float64)
    hd = h.double()
    for t in range(tokens):
        for c in range(top):
            e = int(ids[t, c])
            x = float(weights[t, c]) * hd[t]
            a, b = wgu[e, :ff].double() @ x, wgu[e, ff:].double() @ x
            mid = (a / (1.0 + torch.exp(-a)) * b)
            if dtype == torch.bfloat16:
                mid = mid.to(torch.bfloat16).double()
            want[t] += wd[e].double() @ mid
        want[t] += shared[t].double() / (1.0 + math.exp(-float(gate[t, 1])))
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert float((y - want).abs().max()) <= tol * float(want.abs().max())
    # the same sum formed by the kernel that adds it to the stream and norms the new stream
    x0, w, b = randn(tokens, W, seed=7), randn(W, seed=8), randn(W, seed=9)
    stream = dev(x0.clone())
    rows_out = ops.dynamic_tanh(stream, 0.9, dev(w), dev(b), ops.ChoiceSum(out, dev(h), row_of_pair, dev(weights), True, dev(shared), gate_dev),
                                None, torch.float32).cpu()
    assert torch.allclose(stream.cpu().double(), x0.double() + y, atol=1e-5, rtol=1e-5)
    assert torch.allclose(rows_out.double(), torch.tanh(0.9 * (x0.double() + y)) * w.double() + b.double(), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("tokens,experts,top", [(1, 8, 2), (2, 5, 1), (3, 4, 4)])
@pytest.mark.parametrize("W,ff", [(256, 264), (520, 40), (1024, 320)])
def test_experts_of_steps_with_few_pairs(tokens, experts, top, W, ff):
    """Steps of one to three tokens, whose products are cut along the inner size between a workgroup's wavefronts: inner
    sizes of exactly four steps, of no multiple of a step and of several steps a wavefront; outputs that fill no block."""
    from paged_llm_amd.csrc import ops
    h = (randn(tokens, W, seed=11) * 0.5).to(torch.bfloat16)
    wgu = (randn(experts, 2 * ff, W, seed=12) * W ** -0.5).to(torch.bfloat16)
    wd = (randn(experts, W, ff, seed=13) * ff ** -0.5).to(torch.bfloat16)
    g = torch.Generator().manual_seed(14)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    weights = torch.rand(tokens, top, generator=g) * 0.8 + 0.1
    rows = ops.moe_tile_rows(ids.numel(), experts, torch.bfloat16, W, ff, W)
    assert rows == 16
    sorted_pair, row_of_pair, tiles = ops.moe_align(dev(ids), experts, rows)
    act = ops.moe_expert_gemm(dev(h), dev(wgu), tiles, sorted_pair, top, True, "silu", tile_rows=rows, pair_scale=dev(weights))
    out = ops.moe_expert_gemm(act, dev(wd), tiles, sorted_pair, top, False, tile_rows=rows)
    act, out, where = act.cpu().double(), out.cpu().double(), row_of_pair.cpu().view(tokens, top)
    for t in range(tokens):
        for c in range(top):
            e, row = int(ids[t, c]), int(where[t, c])
            x = float(weights[t, c]) * h[t].double()
            a, b = wgu[e, :ff].double() @ x, wgu[e, ff:].double() @ x
            mid = a / (1.0 + torch.exp(-a)) * b
            assert float((act[row] - mid).abs().max()) <= 1e-2 * float(mid.abs().max()) + 1e-6, ("gated", t, c)
            want = wd[e].double() @ act[row]
            assert float((out[row] - want).abs().max()) <= 1e-5 * float(want.abs().max()) + 1e-7, ("down", t, c)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_preparation_from_float_sums_with_a_latent_of_the_queries(dtype):
    from paged_llm_amd.csrc import ops
    T, rank, q_rank, H, bs = 6, 40, 24, 3, 16
    width = 48
    rows = randn(T, q_rank + rank + H, seed=1)
    wn, wq = randn(rank, seed=2), randn(q_rank, seed=3)
    k_pages = torch.zeros((3, 1, bs, width), dtype=dtype, device="cuda")
    v_pages = torch.zeros((3, 1, width, bs), dtype=dtype, device="cuda")
    q = torch.full((T, H, width), 7.0, dtype=dtype, device="cuda")
    slots = torch.tensor([5, 16, 17, -1, 40, 0], dtype=torch.int32)
    cq = ops.latent_prepare(dev(rows), q_rank, dev(torch.arange(T, dtype=torch.int32)), None, None, dev(wn), 1e-5, dev(slots), k_pages, v_pages, q,
                            H, 8, 0, rank, False, q_latent=(0, q_rank, dev(wq)))

    def normed(x, w):
        return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + 1e-5) * w
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(cq.float().cpu(), normed(rows[:, :q_rank], wq), atol=tol, rtol=tol)
    c = normed(rows[:, q_rank:q_rank + rank], wn)
    for t, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        assert torch.allclose(k_pages[slot // bs, 0, slot % bs, :rank].float().cpu(), c[t], atol=tol, rtol=tol)
        assert torch.allclose(v_pages[slot // bs, 0, :rank, slot % bs].float().cpu(), c[t], atol=tol, rtol=tol)
    assert float(k_pages.float().abs().sum(dim=(1, 3)).view(-1)[[6, 7, 20, 41]].sum()) == 0.0, "slots that nobody wrote stay as they were"
    assert torch.all(q[:, :, rank:] == 0) and torch.all(q[:, :, :rank] == 7.0), "the padding is zeroed, the latent part is left to the next kernel"


@pytest.mark.parametrize("qk_norm", [True, False])
def test_attention_preparation_with_and_without_the_division(qk_norm):
    from paged_llm_amd.csrc import ops
    T, H, G, d, dv, D, bs = 5, 4, 2, 24, 40, 48, 16
    proj = randn(T, (H + G) * d + G * dv, seed=1)
    half = 8
    pos = torch.tensor([0, 1, 2, 7, 30], dtype=torch.int32)
    freq = torch.tensor([10.0 ** (-2.0 * i / 16) for i in range(half)])
    table = torch.arange(32).float()[:, None] * freq[None, :]           # [positions, pairs], as the kernels index it
    angle = table[pos.long()]
    k_pages = torch.zeros((3, G, bs, D), device="cuda")
    v_pages = torch.zeros((3, G, D, bs), device="cuda")
    slots = torch.tensor([0, 1, 2, 20, 47], dtype=torch.int32)
    q = ops.attn_prepare(dev(proj), None, None, None, None, None, None, 1, dev(pos), dev(table.cos().contiguous()), dev(table.sin().contiguous()), 16, False,
                         1e-5, H, G, d, dv, D, torch.float32, dev(slots), k_pages, v_pages, qk_norm=qk_norm).cpu().view(T, H, D)

    def turned(x):
        out = x.clone()
        u, v = x[..., :half], x[..., half:16]
        out[..., :half] = u * angle.cos()[:, None, :] - v * angle.sin()[:, None, :]
        out[..., half:16] = v * angle.cos()[:, None, :] + u * angle.sin()[:, None, :]
        return out / torch.sqrt((out * out).mean(dim=-1, keepdim=True) + 1e-5) if qk_norm else out
    assert torch.allclose(q[:, :, :d], turned(proj[:, :H * d].view(T, H, d)), atol=1e-5, rtol=1e-5) and torch.all(q[:, :, d:] == 0)
    want_k = turned(proj[:, H * d:(H + G) * d].view(T, G, d))
    for t, slot in enumerate(slots.tolist()):
        assert torch.allclose(k_pages[slot // bs, :, slot % bs, :d].cpu(), want_k[t], atol=1e-5, rtol=1e-5)
        assert torch.allclose(v_pages[slot // bs, :, :dv, slot % bs].cpu(), proj[t, (H + G) * d:].view(G, dv), atol=1e-6)
