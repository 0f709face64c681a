"""A plain, slow Nesezen: whole sequences, no cache, no paging, no batches, one function per mechanism.

Nesezen is a pre-norm decoder, x <- x + mixer(N1(x)), x <- x + ff(N2(x)), whose norm computes no statistics:
N(x) = tanh(alpha x) * w + b with a stored scalar alpha.  A layer holds one of three mixers and a dense gated
feed-forward, a mixture of routed experts with a shared one, or no feed-forward; a layer may run with another layer's
weights.

* ``attention``: grouped heads, rotary angles on pairs (i, i + r/2) of the first r elements of a head with the
  frequency rescaling by wavelength (long waves slowed by a factor, short ones kept, a blend between), scores capped by
  c tanh(s / c), a sliding window, softmax.
* ``mlstm``: a matrix memory per head with exponential input gates and sigmoid forget gates held in the log domain
  under a running maximum; the output is divided by max(|n . q|, exp(-m)) and then by its root mean square per head.
* ``latent_attention``: queries through a normed latent, keys and values expanded from one normed latent per token,
  full causal softmax, one sigmoid gate per head on the output.

Everything is computed in one floating type chosen by the caller (float32 by default; float64 to judge which of two
float32 results is closer).  It shares no code with the engine under ``paged-llm_amd/`` and reads ``config.json`` and
the safetensors file on its own.
"""

from __future__ import annotations

import json
import math
import os

import torch


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_weights(model_dir: str) -> dict:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name)
    return out


# --------------------------------------------------------------------------- small pieces
_NOISE = None      # a function applied to every product's operand rows and result (see ``rounding_noise``), or None


def product(x, w, b=None):
    """x W^T (+ b); with ``_NOISE`` set, rows and result are disturbed as a 16-bit compute type would round them."""
    if _NOISE is None:
        y = x @ w.T
        return y if b is None else y + b
    y = _NOISE(x) @ w.T
    return _NOISE(y if b is None else y + b)


class rounding_noise:
    """Inside ``with rounding_noise(seed):`` every product's rows and result are multiplied by 1 + u * 2^-8 with u uniform
    in (-1, 1), drawn from ``seed``: the relative error of two roundings to bfloat16, at random.  Several seeds show how
    far the logits of one position move under the compute type's rounding alone; norms, scores, gates of the recurrence,
    the router and the residual stream stay exact, as the design keeps them in 32 bits."""

    def __init__(self, seed: int, amplitude: float = 2.0 ** -8):
        self.gen = torch.Generator().manual_seed(seed)
        self.amplitude = amplitude

    def __call__(self, t):
        return t * (1.0 + (torch.rand(t.shape, generator=self.gen, dtype=t.dtype) * 2.0 - 1.0) * self.amplitude)

    def __enter__(self):
        global _NOISE
        _NOISE = self
        return self

    def __exit__(self, *exc):
        global _NOISE
        _NOISE = None


def dynamic_tanh(x, alpha, weight, bias):
    """tanh(alpha x) * w + b, element by element: a norm without a mean or a variance."""
    return torch.tanh(alpha * x) * weight + bias


def root_mean_square_norm(x, eps, weight=None):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def log_sigmoid(z):
    """log(1 / (1 + exp(-z))) without overflow on either side."""
    return torch.minimum(z, torch.zeros_like(z)) - torch.log1p(torch.exp(-z.abs()))


def rotary_frequencies(base: float, dims: int, scaling: dict | None) -> list:
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` {factor, low, high, original} by wavelength l = 2 pi / f:
    l < original/high keeps f, l > original/low gives f / factor, between them (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wave = 2.0 * math.pi / f
            if wave > orig / low:
                f = f / factor
            elif wave >= orig / high:
                s = (orig / wave - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, positions, freqs, dims):
    """x [T, heads, d]: element i < dims/2 of every head is paired with element i + dims/2; the pair (u, v) at position p
    becomes (u cos a - v sin a, v cos a + u sin a), a = p f_i formed in float32.  Elements from ``dims`` on pass."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor(freqs, dtype=torch.float32)
    angle = (positions.to(torch.float32)[:, None] * f[None, :]).to(x.dtype)
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def softmax_over_visible(scores, positions, window):
    """Row i keeps the columns j with 0 <= p_i - p_j < window (window 0: every j with p_j <= p_i), softmax over those."""
    d = positions[:, None] - positions[None, :]
    mask = d >= 0
    if window > 0:
        mask = mask & (d < window)
    s = scores.masked_fill(~mask, float("-inf"))
    e = torch.exp(s - s.max(dim=1, keepdim=True).values)
    return e / e.sum(dim=1, keepdim=True)


# --------------------------------------------------------------------------- mixers
def attention_mixer(h, w, m, positions):
    """w: the mixer's tensors by their own names (q, k, v, o); m: its entry of the configuration."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rot = m.get("rot") or {}
    dims = int(rot.get("dims") or 0)
    freqs = rotary_frequencies(rot["base"], dims, rot.get("scaling")) if dims else []
    q = rotate(product(h, w["q"]).view(T, H, d), positions, freqs, dims)
    k = rotate(product(h, w["k"]).view(T, G, d), positions, freqs, dims)
    v = product(h, w["v"]).view(T, G, dv)
    cap = float(m.get("softcap") or 0.0)
    window = int((m.get("mask") or {}).get("size") or 0)
    out = h.new_zeros((T, H, dv))
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        if cap > 0.0:
            s = cap * torch.tanh(s / cap)
        out[:, head] = softmax_over_visible(s, positions, window) @ v[:, g]
    return product(out.reshape(T, H * dv), w["o"])


def mlstm_mixer(h, w, m, eps):
    """Token by token.  Per head: log input gate i = c tanh((W_i h + b_i) / c), log forget gate
    f = logsigmoid(c tanh((W_f h + b_f) / c)); with the running maximum M (0 in front of the sequence)
        M_t = max(f_t + M_(t-1), i_t),   S_t = exp(f_t + M_(t-1) - M_t) S_(t-1) + exp(i_t - M_t) k_t v_t^T,
    n_t the same sum with k_t alone, o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-M_t)) + 1e-6)."""
    T = h.shape[0]
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m.get("gate_cap") or 0.0)
    q = product(h, w["q"]).view(T, H, d) * d ** -0.5
    k = product(h, w["k"]).view(T, H, d)
    v = product(h, w["v"]).view(T, H, dv)
    gi, gf = product(h, w["i"], w["i.b"]), product(h, w["f"], w["f.b"])
    if cap > 0.0:                                            # (a cap of 0 stands for no cap)
        gi, gf = cap * torch.tanh(gi / cap), cap * torch.tanh(gf / cap)
    gf = log_sigmoid(gf)
    S = h.new_zeros((H, d, dv))
    n = h.new_zeros((H, d))
    M = h.new_zeros((H,))
    out = h.new_zeros((T, H, dv))
    for t in range(T):
        M_new = torch.maximum(gf[t] + M, gi[t])
        keep, take = torch.exp(gf[t] + M - M_new), torch.exp(gi[t] - M_new)
        S = keep[:, None, None] * S + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = keep[:, None] * n + take[:, None] * k[t]
        M = M_new
        num = torch.einsum("hnp,hn->hp", S, q[t])
        den = torch.maximum((n * q[t]).sum(dim=1).abs(), torch.exp(-M)) + 1e-6
        out[t] = num / den[:, None]
    u = root_mean_square_norm(out, eps).reshape(T, H * dv) * w["norm"]
    return product(u * torch.sigmoid(product(h, w["g"])), w["o"])


def latent_attention_mixer(h, w, m, eps, positions):
    """c_q = rmsnorm(W_dq h) w_dqn, q = W_uq c_q; c = rmsnorm(W_dkv h) w_dkvn, k = W_uk c, v = W_uv c head by head;
    causal softmax of q . k * scale over all earlier tokens; head h's output times sigmoid((W_g h)_h); W_o."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cq = root_mean_square_norm(product(h, w["dq"]), eps, w["dq.norm"])
    q = product(cq, w["uq"]).view(T, H, d)
    c = root_mean_square_norm(product(h, w["dkv"]), eps, w["dkv.norm"])
    k = product(c, w["uk"]).view(T, H, d)
    v = product(c, w["uv"]).view(T, H, dv)
    gate = torch.sigmoid(product(h, w["g"]))
    out = h.new_zeros((T, H, dv))
    for head in range(H):
        s = (q[:, head] @ k[:, head].T) * float(m["scale"])
        out[:, head] = (softmax_over_visible(s, positions, 0) @ v[:, head]) * gate[:, head:head + 1]
    return product(out.reshape(T, H * dv), w["o"])


# --------------------------------------------------------------------------- feed-forwards
def gated_feed_forward(h, w):
    return product(silu(product(h, w["gate"])) * product(h, w["up"]), w["down"])


def choose_experts(h, router, top):
    """(ids [T, top], weights [T, top]): s = sigmoid(router h), the ``top`` largest (the lower index wins a tie); the weights
    are those s, as they are."""
    s = torch.sigmoid(h @ router.T)
    order = torch.sort(s, dim=1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(s, 1, order)


def routed_feed_forward(h, w, mlp):
    """sum over a token's chosen experts of expert(weight * h), the weight on the expert's input; a shared expert for
    every token, times sigmoid(w_sg . h), on top."""
    T = h.shape[0]
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    ids, weights = choose_experts(h, w["router"], top)
    out = torch.zeros_like(h)
    for t in range(T):
        for c in range(top):
            e = int(ids[t, c])
            we = {n: w[f"e{e}.{n}"] for n in ("gate", "up", "down")}
            out[t] = out[t] + gated_feed_forward((weights[t, c] * h[t])[None, :], we)[0]
    if mlp.get("shared"):
        ws = {n: w[f"shared.{n}"] for n in ("gate", "up", "down")}
        out = out + gated_feed_forward(h, ws) * torch.sigmoid(product(h, w["shared.sg"]))
    return out


# --------------------------------------------------------------------------- the model
def _under(weights: dict, prefix: str, dtype) -> dict:
    return {n[len(prefix) + 1:]: t.to(dtype) for n, t in weights.items() if n.startswith(prefix + ".")}


def _norm(weights, name, x):
    dt = x.dtype
    return dynamic_tanh(x, weights[name + ".alpha"].to(dt), weights[name].to(dt), weights[name + ".b"].to(dt))


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float32, layers_out: list | None = None, positions=None):
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives the residual stream after every layer run."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    positions = torch.arange(T) if positions is None else torch.as_tensor(positions)
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"].to(dtype)[tokens]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of")
        name = f"l{i if src is None else int(src)}"
        m, kind = layer["mixer"], layer["type"]
        wm = _under(weights, name + ".mix", dtype)
        h = _norm(weights, name + ".norm1", x)
        if kind == "attention":
            a = attention_mixer(h, wm, m, positions)
        elif kind == "mlstm":
            a = mlstm_mixer(h, wm, m, eps)
        elif kind == "latent_attention":
            a = latent_attention_mixer(h, wm, m, eps, positions)
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r}")
        x = x + a
        mlp = layer.get("mlp")
        if mlp is not None:
            h = _norm(weights, name + ".norm2", x)
            wf = _under(weights, name + ".mlp", dtype)
            x = x + (gated_feed_forward(h, wf) if mlp["kind"] == "dense" else routed_feed_forward(h, wf, mlp))
        if layers_out is not None:
            layers_out.append(x.clone())
    return product(_norm(weights, "final.norm", x), weights["head"].to(dtype))
