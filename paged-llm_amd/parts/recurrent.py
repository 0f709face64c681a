"""Mixers that carry a state of fixed size per request instead of a growing cache.

Both are the same recurrence per head, S_t = a_t S_(t-1) + k_t (g_t v_t)^T, y_t = S_t^T q_t (+ skip v_t), with S
[N, P] in float in the request's state slot (``ops.linear_recurrence``); they differ in where a, g, k, q and v come from:

* ``mamba2`` (the state-space layer in its dual form): one input product gives a gate z, the values x, the keys B and
  queries C of a few groups that the heads share, and a step size per head; x, B and C pass a short causal convolution
  (whose last inputs are state too) and SiLU; a_t = exp(-exp(A_log) dt_t), g_t = dt_t = softplus(raw + bias), skip = D.
  Behind the recurrence: times silu(z), RMS norm over parts of the channels with a weight, the output product.
* ``retention``: q, k, v and a gate from one product, rotary encoding of q and k (kept in float), k scaled by
  N^(-1/2), a constant decay per head; behind it each head's output divided by its root mean square, times
  silu(gate), the output product.

* ``mlstm`` (a matrix memory with exponential input gates): q, k, v, an output gate and two gate pre-activations per
  head from one product; the log-domain gates i and f run under a running maximum m, which makes a_t =
  exp(f_t + m_(t-1) - m_t) and g_t = exp(i_t - m_t); a normaliser n_t (the same recurrence with k alone) is one more
  column of S; y_t is divided by max(|n_t . q_t|, exp(-m_t)), then by its root mean square per head, times a weight,
  times the sigmoid of the output gate, the output product.

* ``lightning`` (linear attention with a constant decay per head): q, k and v pass SiLU and stay in float from there; no
  positions, no scale; behind the recurrence all heads' outputs are divided by their common root mean square, times a weight,
  times the sigmoid of a gate, the output product.
* ``hgrn2`` (a gated linear recurrence without a key product): the forget gate f, bounded below per channel, decays the
  rows of S one by one, S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T; q passes SiLU; behind it each head's output is divided by
  its root mean square, times a weight that the heads share, the output product.

What enters the recurrence (step sizes, decays, rotated keys and queries, the state) is float whatever the compute type;
the products, the convolution and the activations run in the compute type.  A request's state is zero at its first
token (``ctx.seq_starts == 0``), whatever its slot held before.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Mixer, StateSpec
from .linear import Weight, linear
from .registry import BuildEnv, register_mixer
from .spec import PartSpec, WeightSpec


def _out_dtype(ctx):
    return torch.float32 if getattr(ctx, "float_branch", False) else None


class _StatefulMixer(Mixer):
    graph_capturable = True
    graph_capturable_prompts = True
    MATRICES: tuple = ()

    def _keep(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def assign(self, name, tensor):
        self._keep(name, tensor)


class Mamba2Mixer(_StatefulMixer):
    """params: ``heads``, ``head_dim`` (P), ``state`` (N), ``groups``, ``conv`` (taps), ``norm_groups``, ``eps``.
    Tensors: ``in`` [2 inner + 2 groups N + heads, width] laid out [z | x | B | C | dt], ``conv`` [inner + 2 groups N,
    taps] with ``conv.b``, ``dt_bias``, ``A_log``, ``D`` [heads], ``norm`` [inner], ``o`` [width, inner]."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.P, self.N = int(params["heads"]), int(params["head_dim"]), int(params["state"])
        self.groups, self.taps = int(params.get("groups", 1)), int(params["conv"])
        self.norm_groups, self.eps = int(params.get("norm_groups", 1)), float(params["eps"])
        self.inner = self.heads * self.P
        self.channels = self.inner + 2 * self.groups * self.N
        if self.heads % self.groups or self.inner % self.norm_groups:
            raise ValueError(f"{self.heads} heads in {self.groups} groups, {self.inner} channels normed in {self.norm_groups} parts")
        if not 1 <= self.taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"the convolution kernel takes 1 to {ops.MAX_CONV_TAPS} taps, got {self.taps}")
        self.dtype, self.device = env.dtype, env.device
        self.conv_at = self.heads * self.N * self.P              # the convolution's inputs lie behind S in the slot
        self._w: dict = {}
        self.w_in = self.w_o = None

    def weight_specs(self):
        H = self.heads
        return {"in": WeightSpec((2 * self.inner + 2 * self.groups * self.N + H, self.hidden)),
                "conv": WeightSpec((self.channels, self.taps), role="vector"), "conv.b": WeightSpec((self.channels,), role="vector"),
                "dt_bias": WeightSpec((H,), role="vector"), "A_log": WeightSpec((H,), role="vector"), "D": WeightSpec((H,), role="vector"),
                "norm": WeightSpec((self.inner,), role="vector", init="ones"), "o": WeightSpec((self.hidden, self.inner))}

    def finalize(self):
        self.w_in, self.w_o = Weight(self._w.pop("in")), Weight(self._w.pop("o"))

    def state_spec(self):
        return StateSpec((self.conv_at + self.channels * (self.taps - 1),), torch.float32)

    def forward(self, h, ctx, cache, state):
        w, inner, gn = self._w, self.inner, self.groups * self.N
        proj = linear(h, self.w_in)
        z, xbc, dt_raw = proj[:, :inner], proj[:, inner:inner + self.channels], proj[:, inner + self.channels:]
        seqs = (ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs)
        conv = ops.causal_conv(xbc, w["conv"], w["conv.b"], state, self.conv_at, *seqs, ctx.max_q_len)
        x = conv[:, :inner].unflatten(1, (self.heads, self.P))
        B = conv[:, inner:inner + gn].unflatten(1, (self.groups, self.N))
        C = conv[:, inner + gn:].unflatten(1, (self.groups, self.N))
        if ctx.max_q_len >= ops.RECURRENCE_CHUNKS_FROM:
            # long portions: step sizes and decays by a kernel of their own, all tokens side by side (inside the recurrence
            # their exponentials would stand in every token's way, twice: once per pass over the chunks)
            dt, decay = ops.step_sizes(dt_raw, w["dt_bias"], w["A_log"])
            y = ops.linear_recurrence(C, B, x, decay, state, 0, *seqs, vscale=dt, skip=w["D"], max_q_len=ctx.max_q_len)
        else:
            y = ops.linear_recurrence(C, B, x, None, state, 0, *seqs, skip=w["D"], max_q_len=ctx.max_q_len,
                                      step_sizes=(dt_raw, w["dt_bias"], w["A_log"]))
        u = ops.gated_group_norm(y, z, w["norm"], inner // self.norm_groups, True, self.eps)
        return linear(u, self.w_o, out_dtype=_out_dtype(ctx))


class RetentionMixer(_StatefulMixer):
    """params: ``heads``, ``key_dim`` (N), ``head_dim`` (P), ``decay`` (one number per head), ``position`` (a position
    encoding spec, or None), ``eps``.  Tensors ``q``, ``k`` [heads N, width], ``v``, ``g`` [heads P, width], ``o``."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.N, self.P = int(params["heads"]), int(params["key_dim"]), int(params["head_dim"])
        self.eps = float(params["eps"])
        decay = [float(d) for d in params["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        pos = params.get("position")
        self.position = env.position_encoding(PartSpec(**pos) if isinstance(pos, dict) else pos) if pos else None
        self.dtype, self.device = env.dtype, env.device
        self.decay = torch.tensor(decay, dtype=torch.float32, device=self.device)
        self._w: dict = {}
        self.w_in = self.w_o = None

    def weight_specs(self):
        qk, vg = self.heads * self.N, self.heads * self.P
        return {"q": WeightSpec((qk, self.hidden)), "k": WeightSpec((qk, self.hidden)), "v": WeightSpec((vg, self.hidden)),
                "g": WeightSpec((vg, self.hidden)), "o": WeightSpec((self.hidden, vg))}

    def finalize(self):
        self.w_in = Weight(torch.cat([self._w.pop(n) for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = Weight(self._w.pop("o"))

    def state_spec(self):
        return StateSpec((self.heads * self.N * self.P,), torch.float32)

    def forward(self, h, ctx, cache, state):
        H, N, P = self.heads, self.N, self.P
        rows = linear(h, self.w_in)
        pe = self.position
        rot = (pe.rotary_dim or N) if pe is not None else 0
        tables = (pe.cos, pe.sin) if pe is not None else (ctx.positions.new_zeros((1, 0), dtype=torch.float32),) * 2
        inter = bool(pe.interleaved) if pe is not None else False
        q, k = ops.rotary_to_float(rows, ctx.positions, *tables, H, N, rot, inter, 1.0, second_at=H * N, scale2=N ** -0.5)
        v = rows[:, 2 * H * N:2 * H * N + H * P].unflatten(1, (H, P))
        gate = rows[:, 2 * H * N + H * P:]
        y = ops.linear_recurrence(q, k, v, self.decay, state, 0, ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs,
                                  max_q_len=ctx.max_q_len)
        u = ops.gated_group_norm(y, gate, None, P, False, self.eps)
        return linear(u, self.w_o, out_dtype=_out_dtype(ctx))


class MLstmMixer(_StatefulMixer):
    """A matrix memory per head with exponential input gates and sigmoid forget gates, kept in the log domain:

        i_t = c tanh((W_i h + b_i) / c),   f_t = log sigmoid(c tanh((W_f h + b_f) / c)),   m_t = max(f_t + m_(t-1), i_t),  m_0 = 0
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),   q = W_q h N^(-1/2)

    then each head's o divided by its root mean square, times ``norm`` (a weight over all heads' channels), times
    sigmoid(W_g h), the output product.  The state slot holds S with n as its last column [heads, N, P + 1] and behind
    it m [heads]; gates, maxima, state and what follows the recurrence are float whatever the compute type (the input
    product leaves float sums).

    params: ``heads``, ``key_dim`` (N), ``head_dim`` (P), ``gate_cap`` (c; 0: none), ``eps``.  Tensors ``q``, ``k`` [heads
    N, width], ``v``, ``g`` [heads P, width], ``i``, ``f`` [heads, width] with ``i.b``, ``f.b`` [heads], ``norm`` [heads P],
    ``o`` [width, heads P]."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.N, self.P = int(params["heads"]), int(params["key_dim"]), int(params["head_dim"])
        self.cap, self.eps = float(params.get("gate_cap") or 0.0), float(params["eps"])
        if self.cap < 0.0:
            raise ValueError(f"a cap of the gates is positive (or 0 for none), got {self.cap}")
        self.dtype, self.device = env.dtype, env.device
        self.m_at = self.heads * self.N * (self.P + 1)              # the running maxima lie behind S in the slot
        self._w: dict = {}
        self.w_in = self.w_o = None

    def weight_specs(self):
        H, qk, vg = self.heads, self.heads * self.N, self.heads * self.P
        return {"q": WeightSpec((qk, self.hidden)), "k": WeightSpec((qk, self.hidden)), "v": WeightSpec((vg, self.hidden)),
                "g": WeightSpec((vg, self.hidden)), "i": WeightSpec((H, self.hidden)), "f": WeightSpec((H, self.hidden)),
                "i.b": WeightSpec((H,), role="vector"), "f.b": WeightSpec((H,), role="vector"),
                "norm": WeightSpec((vg,), role="vector", init="ones"), "o": WeightSpec((self.hidden, vg))}

    def finalize(self):
        self.w_in = Weight(torch.cat([self._w.pop(n) for n in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous())
        self.w_o = Weight(self._w.pop("o"))

    def state_spec(self):
        return StateSpec((self.m_at + self.heads,), torch.float32)

    def forward(self, h, ctx, cache, state):
        H, N, P, w = self.heads, self.N, self.P, self._w
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        qk, vg = H * N, H * P
        q = rows[:, :qk].unflatten(1, (H, N))
        k = rows[:, qk:2 * qk].unflatten(1, (H, N))
        v = rows[:, 2 * qk:2 * qk + vg].unflatten(1, (H, P))
        gate = rows[:, 2 * qk + vg:2 * qk + 2 * vg]
        raw_i, raw_f = rows[:, 2 * qk + 2 * vg:2 * qk + 2 * vg + H], rows[:, 2 * qk + 2 * vg + H:]
        seqs = (ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs)
        decay, take, m = ops.mlstm_gates(raw_i, raw_f, w["i.b"], w["f.b"], self.cap, state, self.m_at, *seqs)
        y = ops.linear_recurrence(q, k, v, decay, state, 0, *seqs, vscale=take, max_q_len=ctx.max_q_len, normaliser=True)
        u = ops.mlstm_output(y, m, gate, w["norm"], H, P, N ** -0.5, self.eps, self.dtype)
        return linear(u, self.w_o, out_dtype=_out_dtype(ctx))


class LightningMixer(_StatefulMixer):
    """Linear attention with one constant decay per head:  q = silu(W_q h), k = silu(W_k h), v = silu(W_v h),
    S_t = decay_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t  (no scale, no positions); then all heads' outputs side by side are
    divided by their root mean square, times ``norm``, times sigmoid(W_g h), and projected.  The activated q, k, v, the state
    and the norm are float whatever the compute type.

    params: ``heads``, ``key_dim`` (N), ``head_dim`` (P), ``decay`` (one number per head), ``eps``.  Tensors ``q``, ``k`` [heads N,
    width], ``v``, ``g`` [heads P, width], ``norm`` [heads P], ``o`` [width, heads P]."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.N, self.P = int(params["heads"]), int(params["key_dim"]), int(params["head_dim"])
        self.eps = float(params["eps"])
        decay = [float(d) for d in params["decay"]]
        if len(decay) != self.heads:
            raise ValueError(f"{len(decay)} decays for {self.heads} heads")
        self.dtype, self.device = env.dtype, env.device
        self.decay = torch.tensor(decay, dtype=torch.float32, device=self.device)
        self._w: dict = {}
        self.w_in = self.w_o = None

    def weight_specs(self):
        qk, vg = self.heads * self.N, self.heads * self.P
        return {"q": WeightSpec((qk, self.hidden)), "k": WeightSpec((qk, self.hidden)), "v": WeightSpec((vg, self.hidden)),
                "g": WeightSpec((vg, self.hidden)), "norm": WeightSpec((vg,), role="vector", init="ones"), "o": WeightSpec((self.hidden, vg))}

    def finalize(self):
        self.w_in = Weight(torch.cat([self._w.pop(n) for n in ("q", "k", "v", "g")], dim=0).contiguous())
        self.w_o = Weight(self._w.pop("o"))

    def state_spec(self):
        return StateSpec((self.heads * self.N * self.P,), torch.float32)

    def forward(self, h, ctx, cache, state):
        H, N, P = self.heads, self.N, self.P
        rows = linear(h, self.w_in)
        qk, vg = H * N, H * P
        acts = ops.silu_to_float(rows, 2 * qk + vg)
        q, k = acts[:, :qk].unflatten(1, (H, N)), acts[:, qk:2 * qk].unflatten(1, (H, N))
        v = acts[:, 2 * qk:].unflatten(1, (H, P))
        y = ops.linear_recurrence(q, k, v, self.decay, state, 0, ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs,
                                  max_q_len=ctx.max_q_len)
        u = ops.gated_group_norm(y, rows[:, 2 * qk + vg:], self._w["norm"], vg, False, self.eps, gate_activation="sigmoid")
        return linear(u, self.w_o, out_dtype=_out_dtype(ctx))


class Hgrn2Mixer(_StatefulMixer):
    """A gated linear recurrence whose forget gate also decides what is written:  q = silu(W_q h), v = W_v h,
    f = l + (1 - l) sigmoid(W_f h + b_f) per head and channel with a stored lower bound l,
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,  o_t = S_t^T q_t;  then each head's o divided by its root mean square, times
    ``norm`` (one weight over a head's channels, shared by the heads), the output product.  Gates, decays, the state and the
    norm are float whatever the compute type (the input product leaves float sums).

    params: ``heads``, ``key_dim`` (N), ``head_dim`` (P), ``eps``.  Tensors ``q``, ``f`` [heads N, width], ``f.b``, ``lower`` [heads N],
    ``v`` [heads P, width], ``norm`` [P], ``o`` [width, heads P]."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.N, self.P = int(params["heads"]), int(params["key_dim"]), int(params["head_dim"])
        self.eps = float(params["eps"])
        self.dtype, self.device = env.dtype, env.device
        self._w: dict = {}
        self.w_in = self.w_o = self.norm_w = None

    def weight_specs(self):
        qf, v = self.heads * self.N, self.heads * self.P
        return {"q": WeightSpec((qf, self.hidden)), "f": WeightSpec((qf, self.hidden)), "f.b": WeightSpec((qf,), role="vector"),
                "lower": WeightSpec((qf,), role="vector", init="zeros"), "v": WeightSpec((v, self.hidden)),
                "norm": WeightSpec((self.P,), role="vector", init="ones"), "o": WeightSpec((self.hidden, v))}

    def finalize(self):
        self.w_in = Weight(torch.cat([self._w.pop(n) for n in ("q", "f", "v")], dim=0).contiguous())
        self.w_o = Weight(self._w.pop("o"))
        self.norm_w = self._w.pop("norm").repeat(self.heads).contiguous()       # the heads share one weight

    def state_spec(self):
        return StateSpec((self.heads * self.N * self.P,), torch.float32)

    def forward(self, h, ctx, cache, state):
        H, N, P = self.heads, self.N, self.P
        rows = linear(h, self.w_in, out_dtype=torch.float32)
        qkf = ops.bounded_forget_gates(rows, self._w["f.b"], self._w["lower"], H * N)
        q, k, f = (qkf[i].unflatten(1, (H, N)) for i in range(3))
        v = rows[:, 2 * H * N:].unflatten(1, (H, P))
        y = ops.linear_recurrence(q, k, v, None, state, 0, ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs,
                                  max_q_len=ctx.max_q_len, row_decay=f)
        u = ops.gated_group_norm(y, None, self.norm_w, P, False, self.eps, gate_activation=None, out_dtype=self.dtype)
        return linear(u, self.w_o, out_dtype=_out_dtype(ctx))


register_mixer("lightning", LightningMixer)
register_mixer("hgrn2", Hgrn2Mixer)
register_mixer("mamba2", Mamba2Mixer)
register_mixer("retention", RetentionMixer)
register_mixer("mlstm", MLstmMixer)
