"""A plain, slow Renadra: whole sequences, no cache, no paging, no batches, one function per mechanism.

Renadra is a pre-norm decoder over RMS norms, x <- x + mixer(N1(x)), x <- x + ff(N2(x)), with a gated feed-forward in
every layer that has one.  The embedding adds a hashed bigram row to the scaled token row; a range of layers may run
several times with the same weights, the embedding's output added to the stream in front of every pass but the first.
A layer holds one of three mixers:

* ``parallel``: two mixers read the same rows and their outputs are added with a factor each.  The left one is
  attention without a softmax (every visible key weighs sigmoid(capped score + a per-head number)), the values being
  the keys before their rotation, under a sliding window that also keeps the sequence's first positions, with
  half-split rotary pairs whose frequencies are blended by wavelength and whose tables carry a factor.  The right one
  is a linear recurrence with a constant decay per head over SiLU-activated q, k and v, normed over all heads and
  gated.
* ``attention``: grouped heads with biases, interleaved rotary pairs, values divided by their root mean square, a
  sliding window, softmax.
* ``hgrn2``: a linear recurrence whose forget gate (bounded below per channel) decays the rows and whose complement is
  the key.

Everything is computed in one floating type chosen by the caller.  It shares no code with the engine under
``paged-llm_amd/``.
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
def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


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
    far the logits of one position move under the compute type's rounding alone; norms, scores, the recurrences' gates
    and states and the residual stream stay exact, as the design keeps them in 32 bits."""

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


def bigram_rows(tokens, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the bigram table per position: a hash of the token before and the token itself, the table's last row
    (number ``buckets``) where there is no token before."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((int(prev) * mul_prev + int(cur) * mul_cur) % buckets)
    return rows


def embedding(tokens, embed, bigram, scale: float, hashing: dict | None):
    x = embed[torch.tensor(list(tokens))] * scale
    if hashing:
        x = x + bigram[torch.tensor(bigram_rows(list(tokens), int(hashing["buckets"]), int(hashing["mul_prev"]), int(hashing["mul_cur"])))]
    return x


# --------------------------------------------------------------------------- rotations
def frequencies(dims: int, base: float, scaling: dict | None):
    """(frequencies of the dims/2 pairs in float64, factor on the tables).  With ``scaling``: a pair's frequency is
    blended between itself and itself / factor by where its index lies between the indices whose wavelengths make
    ``fast`` and ``slow`` turns over ``original`` positions."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=torch.float64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, dims: int, base: float, interleaved: bool, scaling: dict | None = None):
    """x [T, heads, d]: the first ``dims`` elements of every head turned by position * frequency; pairs (i, i + dims/2)
    or, ``interleaved``, (2i, 2i + 1)."""
    if dims <= 0:
        return x
    f, mag = frequencies(dims, base, scaling)
    ang = (torch.tensor(list(positions), dtype=torch.float64)[:, None] * f[None, :])
    cos, sin = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    half = dims // 2
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


def visible(T: int, size: int, keep_first: int = 0):
    """[T, T] bool: query i sees key j when j <= i and (i - j < size or j < keep_first); size 0: every j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = (i - j < size) if size > 0 else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


# --------------------------------------------------------------------------- mixers
def sigmoid_attention(h, w: dict, m: dict, positions):
    """The left side of ``parallel``: no softmax, values = keys before rotation."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"])
    q = product(h, w["q"], w["q.b"]).view(T, H, d)
    k = product(h, w["k"], w["k.b"]).view(T, G, d)
    v = k
    rot = m.get("rot") or {}
    dims = int(rot.get("dims") or 0)
    if dims:
        q = rotate(q, positions, dims, float(rot["base"]), False, rot.get("scaling"))
        k = rotate(k, positions, dims, float(rot["base"]), False, rot.get("scaling"))
    mask = m.get("mask") or {}
    see = visible(T, int(mask.get("size") or 0), int(mask.get("keep_first") or 0))
    cap = float(m.get("softcap") or 0.0)
    out = torch.zeros(T, H, v.shape[-1], dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        p = torch.sigmoid(s + w["pb"][head]) * see
        out[:, head] = p @ v[:, g]
    return product(out.reshape(T, -1), w["o"])


def lightning_attention(h, w: dict, m: dict, eps: float):
    """The right side of ``parallel``: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, token by token."""
    T = h.shape[0]
    H, N, P = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(product(h, w["q"])).view(T, H, N)
    k = silu(product(h, w["k"])).view(T, H, N)
    v = silu(product(h, w["v"])).view(T, H, P)
    decay = [float(a) for a in m["decay"]]
    o = torch.zeros(T, H, P, dtype=h.dtype)
    for head in range(H):
        S = torch.zeros(N, P, dtype=h.dtype)
        for t in range(T):
            S = decay[head] * S + torch.outer(k[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    u = rms_norm(o.reshape(T, H * P), w["norm"], eps) * torch.sigmoid(product(h, w["g"]))
    return product(u, w["o"])


def parallel(h, w: dict, m: dict, eps: float, positions):
    left = sigmoid_attention(h, {k[5:]: t for k, t in w.items() if k.startswith("left.")}, m["left"], positions)
    right = lightning_attention(h, {k[6:]: t for k, t in w.items() if k.startswith("right.")}, m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def attention(h, w: dict, m: dict, eps: float, positions):
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"])
    q = product(h, w["q"], w["q.b"]).view(T, H, d)
    k = product(h, w["k"], w["k.b"]).view(T, G, d)
    v = rms_norm(product(h, w["v"], w["v.b"]).view(T, G, dv), None, eps)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims") or 0)
    if dims:
        q = rotate(q, positions, dims, float(rot["base"]), True)
        k = rotate(k, positions, dims, float(rot["base"]), True)
    see = visible(T, int((m.get("mask") or {}).get("size") or 0))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        s = s.masked_fill(~see, float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    return product(out.reshape(T, -1), w["o"], w["o.b"])


def hgrn2(h, w: dict, m: dict, eps: float):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t per head; f = l + (1 - l) sigmoid(W_f h + b)."""
    T = h.shape[0]
    H, N, P = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(product(h, w["q"])).view(T, H, N)
    v = product(h, w["v"]).view(T, H, P)
    low = w["lower"]
    f = (low + (1.0 - low) * torch.sigmoid(product(h, w["f"], w["f.b"]))).view(T, H, N)
    o = torch.zeros(T, H, P, dtype=h.dtype)
    for head in range(H):
        S = torch.zeros(N, P, dtype=h.dtype)
        for t in range(T):
            S = f[t, head][:, None] * S + torch.outer(1.0 - f[t, head], v[t, head])
            o[t, head] = S.T @ q[t, head]
    u = rms_norm(o, w["norm"], eps).reshape(T, H * P)
    return product(u, w["o"])


def gated_mlp(h, w: dict):
    return product(silu(product(h, w["gate"])) * product(h, w["up"]), w["down"])


# --------------------------------------------------------------------------- the model
def run_order(cfg: dict) -> list:
    """[(layer, whether a pass of the repeated range other than the first starts here)]."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for p in range(times):
        order += [(i, p > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float32, layer_outputs: list | None = None):
    """Logits [T, vocab] of one sequence from its first token on.  ``layer_outputs``: a list that receives the stream
    after every layer run."""
    with torch.no_grad():
        return _forward(cfg, weights, tokens, dtype, layer_outputs)


def _forward(cfg, weights, tokens, dtype, layer_outputs):
    W = {k: (t.to(dtype) if t.is_floating_point() else t) for k, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    emb = cfg.get("embedding") or {}
    x0 = embedding(tokens, W["embed"], W.get("bigram"), float(emb.get("scale") or 1.0), emb.get("bigram"))
    x = x0.clone()
    positions = list(range(len(tokens)))
    for i, again in run_order(cfg):
        layer = cfg["layers"][i]
        if again:
            x = x + x0
        w = {k[len(f"l{i}.mix."):]: t for k, t in W.items() if k.startswith(f"l{i}.mix.")}
        h = rms_norm(x, W[f"l{i}.norm1"], eps)
        if layer["type"] == "parallel":
            a = parallel(h, w, layer["mixer"], eps, positions)
        elif layer["type"] == "attention":
            a = attention(h, w, layer["mixer"], eps, positions)
        elif layer["type"] == "hgrn2":
            a = hgrn2(h, w, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + a
        if layer.get("mlp"):
            w = {k[len(f"l{i}.mlp."):]: t for k, t in W.items() if k.startswith(f"l{i}.mlp.")}
            x = x + gated_mlp(rms_norm(x, W[f"l{i}.norm2"], eps), w)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return product(rms_norm(x, W["final.norm"], eps), W["head"])
