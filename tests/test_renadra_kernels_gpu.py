"""The kernels that came with Renadra, each against a plain PyTorch float32 (or float64) version of the same operation:
attention without a softmax on the matrix cores and in the plain kernel (sigmoid weights, a cap, a window beside kept
first positions), kept first positions under a softmax, the attention preparation's value modes, the recurrence with a
decay per state row (token by token and in chunks), the bounded forget gates, the activation into float rows, the gate
activations of the norm behind a recurrence, the bigram embedding with its carried token, the pre-norm sum in the RMS
kernel and the scaled sum of two branches."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(t):
    return t.to("cuda")


def randn(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32).to(dtype)


class _Ctx:
    capturing = False
    graph_layout = None

    def __init__(self, q_lens, k_lens):
        self.q_lens, self.k_lens, self.num_seqs = q_lens, k_lens, len(q_lens)
        self.max_q_len, self.max_k_len = max(q_lens), max(k_lens)
        self.launch_cache = {}


def _paged_case(q_lens, k_lens, H, G, D, bs, dtype, seed):
    """Random queries, keys and values laid out in pages in a shuffled order; returns the device operands and the float
    copies per sequence."""
    T, S = sum(q_lens), len(q_lens)
    q = (randn(T, H * D, seed=seed) * 0.5).to(dtype)
    pages_per = [-(-k // bs) for k in k_lens]
    total = sum(pages_per) + 3
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed + 1)).tolist()
    k_pages = (randn(total, G, bs, D, seed=seed + 2) * 7.0).to(dtype)           # what no table names is large, and must not show
    v_pages = (randn(total, G, D, bs, seed=seed + 3) * 7.0).to(dtype)
    tables = torch.zeros(S, max(pages_per), dtype=torch.int32)
    keys, values, at = [], [], 0
    for s in range(S):
        k = (randn(k_lens[s], G, D, seed=seed + 10 + s) * 0.7).to(dtype)
        v = randn(k_lens[s], G, D, seed=seed + 40 + s).to(dtype)
        keys.append(k.float()); values.append(v.float())
        for p in range(pages_per[s]):
            page = perm[at]; at += 1
            tables[s, p] = page
            n = min(bs, k_lens[s] - p * bs)
            k_pages[page, :, :n] = k[p * bs:p * bs + n].transpose(0, 1)
            v_pages[page, :, :, :n] = v[p * bs:p * bs + n].permute(1, 2, 0)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    return q, k_pages, v_pages, tables, cu, torch.tensor(k_lens, dtype=torch.int32), keys, values


def _plain_attention(q, keys, values, q_lens, k_lens, H, G, D, scale, window, keep, cap, bias, sigmoid):
    out = torch.zeros(sum(q_lens), H, D, dtype=torch.float64)
    at = 0
    for s, (nq, nk) in enumerate(zip(q_lens, k_lens)):
        for i in range(nq):
            pos = nk - nq + i
            js = [j for j in range(pos + 1) if window == 0 or pos - j < window or j < keep]
            for h in range(H):
                qv = q[at + i].double().view(H, D)[h]
                sc = torch.stack([qv @ keys[s][j, h // (H // G)].double() for j in js]) * scale
                if cap > 0:
                    sc = cap * torch.tanh(sc / cap)
                w = torch.sigmoid(sc + (float(bias[h]) if bias is not None else 0.0)) if sigmoid else torch.softmax(sc, 0)
                out[at + i, h] = sum(w[n] * values[s][j, h // (H // G)].double() for n, j in enumerate(js))
        at += nq
    return out.view(-1, H * D)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("q_lens,k_lens", [([1, 1, 1], [150, 3, 64]), ([37, 1, 2], [37, 200, 130]), ([70], [135])])
@pytest.mark.parametrize("H,G,D", [(4, 2, 16), (8, 1, 64), (3, 3, 96), (2, 1, 128)])
@pytest.mark.parametrize("window,keep,cap", [(0, 0, 0.0), (40, 0, 5.0), (33, 5, 20.0), (16, 70, 0.0), (1, 1, 3.0)])
def test_attention_with_sigmoid_weights(dtype, q_lens, k_lens, H, G, D, window, keep, cap):
    """Decode steps, mixed steps and a prompt portion; the matrix-core kernel in bfloat16, the plain one in float32."""
    from paged_llm_amd.csrc import ops
    if window == 0:
        keep = 0
    q, kp, vp, tables, cu, lens, keys, values = _paged_case(q_lens, k_lens, H, G, D, 16, dtype, seed=H * 100 + D + window)
    bias = randn(H, seed=9)
    weights = ops.KeyWeights(keep, True, dev(bias))
    got = ops.paged_attention(dev(q), dev(kp), dev(vp), dev(tables), dev(cu), dev(lens), H, G, D, 0.3, window, _Ctx(q_lens, k_lens),
                              terms=ops.ScoreTerms(cap) if cap else None, weights=weights)
    want = _plain_attention(q, keys, values, q_lens, k_lens, H, G, D, 0.3, window, keep, cap, bias, True)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    err = float((got.double().cpu() - want).abs().max() / want.abs().max())
    assert err < tol, err


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("window,keep", [(20, 3), (16, 40)])
def test_kept_first_positions_under_a_softmax(dtype, window, keep):
    from paged_llm_amd.csrc import ops
    q_lens, k_lens, H, G, D = [5, 1], [90, 131], 4, 2, 32
    q, kp, vp, tables, cu, lens, keys, values = _paged_case(q_lens, k_lens, H, G, D, 16, dtype, seed=77)
    got = ops.paged_attention(dev(q), dev(kp), dev(vp), dev(tables), dev(cu), dev(lens), H, G, D, 0.3, window, _Ctx(q_lens, k_lens),
                              weights=ops.KeyWeights(keep, False, None))
    want = _plain_attention(q, keys, values, q_lens, k_lens, H, G, D, 0.3, window, keep, 0.0, None, False)
    assert float((got.double().cpu() - want).abs().max() / want.abs().max()) < (2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("values", ["projected", "normed", "keys"])
def test_attention_preparation_value_modes(values):
    """What lands in the value pages: the product's value columns, those divided by their root mean square, or the keys as
    they were before their rotation (bias included)."""
    from paged_llm_amd.csrc import ops
    T, H, G, d, bs = 9, 4, 2, 16, 16
    dv = d if values == "keys" else 24
    D = 32
    channels = (H + G) * d + (0 if values == "keys" else G * dv)
    proj, bias = randn(T, channels + 3, seed=1), randn(channels, seed=2)
    pos = torch.arange(T, dtype=torch.int32) + 4
    ang = torch.outer(torch.arange(64, dtype=torch.float32), torch.tensor([1.0, 0.3, 0.1, 0.01]))
    cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
    kp, vp = torch.zeros(2, G, bs, D), torch.zeros(2, G, D, bs)
    slots = torch.arange(T, dtype=torch.int32) + 5
    k_pages, v_pages = dev(kp), dev(vp)
    ops.attn_prepare(dev(proj), dev(bias), None, None, None, None, None, 1, dev(pos), dev(cos), dev(sin), 8, False, 1e-3, H, G, d, dv, D,
                     torch.float32, dev(slots), k_pages, v_pages, qk_norm=False, values=values)
    x = proj[:, :channels] + bias
    k = x[:, H * d:(H + G) * d].view(T, G, d)
    v = k if values == "keys" else x[:, (H + G) * d:].view(T, G, dv)
    if values == "normed":
        v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-3)
    for t in range(T):
        slot = int(slots[t])
        got = v_pages[slot // bs, :, :, slot % bs].cpu()
        assert torch.allclose(got[:, :dv], v[t], atol=1e-6, rtol=1e-6) and float(got[:, dv:].abs().max() if dv < D else 0.0) == 0.0
        gk = k_pages[slot // bs, :, slot % bs].cpu()
        assert torch.allclose(gk[:, 8:d], k[t][:, 8:], atol=1e-6) and not torch.allclose(gk[:, :8], k[t][:, :8], atol=1e-3)


def _plain_row_recurrence(q, k, v, f, S):
    """S [H, N, P] moved token by token; returns the outputs [T, H, P] and the last S."""
    outs = []
    for t in range(q.shape[0]):
        S = f[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        outs.append(torch.einsum("hnp,hn->hp", S, q[t]))
    return torch.stack(outs) if outs else torch.zeros(0, *S.shape[::2]), S


@pytest.mark.parametrize("H,N,P", [(2, 32, 32), (1, 70, 66), (3, 16, 100), (2, 128, 128)])
@pytest.mark.parametrize("long", [False, True])
def test_recurrence_with_a_decay_per_row(H, N, P, long):
    """Three sequences (one that starts, one that goes on from a stored state, one without tokens) against the recurrence token
    by token in float64; ``long``: portions that run in chunks side by side."""
    from paged_llm_amd.csrc import ops
    lens, starts = ([300, 0, 141, 5] if long else [9, 0, 1, 30]), [0, 3, 7, 2]
    T = sum(lens)
    qkf = randn(3, T, H * N, seed=1)
    qkf[2] = torch.sigmoid(qkf[2] * 2.0 + 2.0)
    qkf[1] = 1.0 - qkf[2]
    v = randn(T, H * P + 7, seed=2)
    state = randn(6, H * N * P + 11, seed=3) * 0.3
    slots = torch.tensor([4, 0, 2, 1], dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    st, dq = dev(state.clone()), dev(qkf)
    y = ops.linear_recurrence(dq[0].unflatten(1, (H, N)), dq[1].unflatten(1, (H, N)), dev(v)[:, 3:3 + H * P].unflatten(1, (H, P)), None, st, 5,
                              dev(slots), dev(torch.tensor(starts, dtype=torch.int32)), dev(cu), 4, max_q_len=max(lens), row_decay=dq[2].unflatten(1, (H, N)))
    for s, n in enumerate(lens):
        a, b = int(cu[s]), int(cu[s + 1])
        S0 = state[slots[s], 5:5 + H * N * P].double().view(H, N, P) if starts[s] > 0 else torch.zeros(H, N, P, dtype=torch.float64)
        q, k, f = (qkf[i, a:b].double().view(n, H, N) for i in range(3))
        want, S1 = _plain_row_recurrence(q, k, v[a:b, 3:3 + H * P].double().view(n, H, P), f, S0)
        if n:
            assert float((y[a:b].double().cpu().view(n, H, P) - want).abs().max()) < 2e-4 * max(1.0, float(want.abs().max()))
            assert float((st[slots[s], 5:5 + H * N * P].double().cpu().view(H, N, P) - S1).abs().max()) < 2e-4 * max(1.0, float(S1.abs().max()))
        else:
            assert torch.equal(st[slots[s]].cpu(), state[slots[s]])
    assert torch.equal(st[:, :5].cpu(), state[:, :5]) and torch.equal(st[:, 5 + H * N * P:].cpu(), state[:, 5 + H * N * P:])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bounded_forget_gates_and_activated_rows(dtype):
    from paged_llm_amd.csrc import ops
    T, C = 13, 40
    rows = (randn(T, 2 * C + 9, seed=1) * 3.0).to(dtype)
    bias, lower = randn(C, seed=2), torch.rand(C, generator=torch.Generator().manual_seed(3))
    got = ops.bounded_forget_gates(dev(rows), dev(bias), dev(lower), C).cpu()
    r = rows.float()
    f = lower + (1 - lower) * torch.sigmoid(r[:, C:2 * C] + bias)
    assert torch.allclose(got[0], r[:, :C] * torch.sigmoid(r[:, :C]), atol=1e-6, rtol=1e-5)
    assert torch.allclose(got[2], f, atol=1e-6, rtol=1e-6) and torch.allclose(got[1], 1 - f, atol=1e-6, rtol=1e-6)
    assert bool((got[2] >= lower - 1e-7).all()) and bool((got[2] <= 1.0).all())
    act = ops.silu_to_float(dev(rows)[:, 2:], 31).cpu()
    assert act.dtype == torch.float32 and torch.allclose(act, r[:, 2:33] * torch.sigmoid(r[:, 2:33]), atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inner,group", [(192, 192), (96, 32), (100, 50), (2048, 128)])
def test_norm_behind_a_recurrence_with_a_sigmoid_gate_and_without_a_gate(inner, group, out_dtype):
    from paged_llm_amd.csrc import ops
    T = 6
    y, gate, w = randn(T, inner, seed=1) * 3.0, randn(T, inner + 8, seed=2).to(out_dtype), randn(inner, seed=3)
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2
    yn = (y.view(T, -1, group) / torch.sqrt((y.view(T, -1, group) ** 2).mean(-1, keepdim=True) + 1e-4)).view(T, inner)
    got = ops.gated_group_norm(dev(y), dev(gate)[:, 4:4 + inner], dev(w), group, False, 1e-4, gate_activation="sigmoid")
    assert got.dtype == out_dtype and torch.allclose(got.float().cpu(), yn * torch.sigmoid(gate[:, 4:4 + inner].float()) * w, atol=tol, rtol=tol)
    got = ops.gated_group_norm(dev(y), None, dev(w), group, False, 1e-4, gate_activation=None, out_dtype=out_dtype)
    assert got.dtype == out_dtype and torch.allclose(got.float().cpu(), yn * w, atol=tol, rtol=tol)
    got = ops.gated_group_norm(dev(y), dev(gate)[:, :inner], dev(w), group, False, 1e-4)
    g = gate[:, :inner].float()
    assert torch.allclose(got.float().cpu(), yn * (g * torch.sigmoid(g)) * w, atol=tol, rtol=tol), "the SiLU gate is as it was"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bigram_embedding_carries_the_token_before(dtype):
    """Two steps: the second one's first rows take the pairs with the tokens the first step ended on; a sequence that starts
    takes the table's last row whatever its slot holds; a second gather of the same step leaves the state alone."""
    from paged_llm_amd.csrc import ops
    V, Hd, buckets, mp, mc = 50, 24, 13, 1000003, 7
    table, pairs = randn(V, Hd, seed=1).to(dtype), randn(buckets + 1, Hd, seed=2).to(dtype)
    state = dev(torch.full((4, 1), 41, dtype=torch.int32))
    def run(ids, lens, starts, slots, again=False, rows=None):
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        rows = rows if rows is not None else dev(torch.zeros(len(ids), dtype=torch.int32))
        x = ops.embed_bigram(dev(torch.tensor(ids, dtype=torch.int32)), dev(table), dev(pairs), 0.5, buckets, mp, mc, state,
                             dev(torch.tensor(slots, dtype=torch.int32)), dev(torch.tensor(starts, dtype=torch.int32)), dev(cu), len(lens), rows,
                             move_state=not again)
        return x.cpu(), rows
    def want(ids, prevs):
        out = []
        for t, p in zip(ids, prevs):
            row = buckets if p is None else (p * mp + t * mc) % buckets
            out.append(table[t].float() * 0.5 + pairs[row].float())
        return torch.stack(out)
    ids = [3, 9, 9, 4, 17, 30]
    x, rows = run(ids, [4, 0, 2], [0, 5, 0], [2, 1, 0])
    assert torch.allclose(x, want(ids, [None, 3, 9, 9, None, 17]), atol=1e-6)
    assert state.cpu().view(-1).tolist() == [30, 41, 4, 41]
    again, _ = run(ids, [4, 0, 2], [0, 5, 0], [2, 1, 0], again=True, rows=rows)
    assert torch.equal(again, x) and state.cpu().view(-1).tolist() == [30, 41, 4, 41]
    ids2 = [8, 1, 2, 5]
    x2, _ = run(ids2, [1, 2, 1], [4, 7, 0], [2, 3, 0])
    assert torch.allclose(x2, want(ids2, [4, 41, 1, None]), atol=1e-6)
    assert state.cpu().view(-1).tolist() == [5, 41, 8, 2]


@pytest.mark.parametrize("hidden", [50, 192, 2048, 4100])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_pre_norm_sum_in_the_rms_kernel(hidden, out_dtype):
    from paged_llm_amd.csrc import ops
    x, d, w = randn(5, hidden, seed=1) * 2.0, randn(5, hidden, seed=2), randn(hidden, seed=3)
    stream = dev(x.clone())
    got = ops.rms_sandwich(stream, dev(d), None, 1.0, 1e-5, w_next=dev(w), out_dtype=out_dtype)
    assert torch.equal(stream.cpu(), x + d), "the residual sum is one float addition"
    s = x + d
    tol = 1e-5 if out_dtype == torch.float32 else 1e-2
    assert torch.allclose(got.float().cpu(), s / torch.sqrt((s * s).mean(-1, keepdim=True) + 1e-5) * w, atol=tol, rtol=tol)
    a, b = dev(x), dev(d)
    assert torch.allclose(ops.scaled_sum(a, 0.8, b, -1.25).cpu(), 0.8 * x - 1.25 * d, atol=1e-6)
    # a branch that is the weighted sum of two, formed by the same kernel
    e = randn(5, hidden, seed=4)
    stream = dev(x.clone())
    got = ops.rms_sandwich(stream, ops.WeightedPair(dev(d), 0.7, dev(e), 1.2), None, 1.0, 1e-5, w_next=dev(w), out_dtype=out_dtype)
    s = x + (0.7 * d + 1.2 * e)
    assert torch.allclose(stream.cpu(), s, atol=1e-6, rtol=1e-6)
    assert torch.allclose(got.float().cpu(), s / torch.sqrt((s * s).mean(-1, keepdim=True) + 1e-5) * w, atol=tol, rtol=tol)
    stream = dev(x.clone())
    ops.stream_add(stream, ops.WeightedPair(dev(d), 0.7, dev(e), 1.2))
    assert torch.allclose(stream.cpu(), s, atol=1e-6, rtol=1e-6)
