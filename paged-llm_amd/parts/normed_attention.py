"""Causal attention over the paged cache whose queries and keys are prepared in float between the input product and the
pages: usually divided by their root mean square per head (``qk_norm``; a layer may switch that off and keep the rest).

q, k, v (and one gate per head) from one product of the mixer's input -> optional biases -> optional short causal
convolution over time on every channel of q, k and v (the last taps - 1 projected rows of a request are its state) ->
rotary encoding of q and k -> q and k of every head divided by their root mean square (an RMS norm without a weight) ->
k and v into their pages -> attention with a causal mask that is full, a sliding window, or blocks of positions counted
from position 0 (a query sees the keys of its own block only), optionally with a learned logit per head in the softmax's
denominator -> optionally every head's output times the sigmoid of its gate -> output product, optionally with a bias.

Keys and values may differ in width: pages and query rows hold heads of D = max(key, value) elements rounded up to a
multiple of 16, the rest zero, and the paged attention kernels (matrix-core ones in bfloat16, the plain one in float32)
serve the layer at head size D.  What lies between the products is float: the input product leaves float sums, one
kernel does bias, convolution, rotation, norm and the cache write from them.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import BLOCK, CacheSpec, Mixer, PageTensor, StateSpec
from .linear import Weight, linear
from .registry import BuildEnv, register_mixer
from .spec import PartSpec, WeightSpec

MASKS = ("full", "window", "chunk")


class NormedAttention(Mixer):
    """params: ``heads``, ``kv_heads``, ``key_dim``, ``value_dim``, ``scale``, ``eps`` (of the q/k norm), ``position`` (a
    rotary spec or None), ``mask`` ("full", "window" or "chunk") with ``mask_size``, ``conv`` (taps of the convolution
    over time; 0: none), ``bias`` (q, k, v and the output product have biases), ``sinks`` (a logit per head in the
    softmax's sum), ``head_gate`` (a gate per head from the mixer's input), ``qk_norm`` (default True; False: q and k go
    to the scores as they are rotated), ``score_cap`` c > 0 (the scaled product x becomes c tanh(x / c); default none);
    ``output_bias`` (default: as ``bias``; False: the projections have biases, the output product has none);
    ``values``: "projected" (default), "normed" (every value head divided by its root mean square, ``eps`` inside the root, no
    weight, and cached so) or "keys" (there is no value product: a value head is its key head as projected, before the
    rotation; the two sizes are equal); ``keep_first`` (with a window: the sequence's first positions that every later query
    still sees, at their own positions); ``weighting``: "softmax" (default) or "sigmoid" (a visible key weighs
    sigmoid(score + ``pb``[head]), not normalised over the keys).  Tensors (under the part's prefix): ``q``,
    ``k``, ``v``, ``o``; ``q.b``, ``k.b``, ``v.b``, ``o.b``; ``q.conv``, ``k.conv``, ``v.conv`` [channels, taps];
    ``sink`` [heads]; ``g`` [heads, width]; ``pb`` [heads]."""
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.kv_heads = int(params["heads"]), int(params.get("kv_heads") or params["heads"])
        self.d, self.dv = int(params["key_dim"]), int(params["value_dim"])
        self.scale, self.eps = float(params["scale"]), float(params["eps"])
        self.mask, self.mask_size = params.get("mask") or "full", int(params.get("mask_size") or 0)
        self.has_conv = int(params.get("conv") or 0) >= 1
        self.taps = max(1, int(params.get("conv") or 1))
        self.bias, self.has_sinks, self.head_gate = bool(params.get("bias")), bool(params.get("sinks")), bool(params.get("head_gate"))
        self.qk_norm, self.score_cap = bool(params.get("qk_norm", True)), float(params.get("score_cap") or 0.0)
        self.out_bias = bool(params.get("output_bias", self.bias))
        self.values = params.get("values") or "projected"
        self.keep_first = int(params.get("keep_first") or 0)
        self.weighting = params.get("weighting") or "softmax"
        if self.values not in ops.VALUE_MODES or self.weighting not in ("softmax", "sigmoid"):
            raise ValueError(f"values {self.values!r}: one of {tuple(ops.VALUE_MODES)}; weighting {self.weighting!r}: softmax or sigmoid")
        if self.values == "keys" and self.d != self.dv:
            raise ValueError(f"values that are the keys have the keys' size: {self.dv} against {self.d}")
        if self.keep_first < 0 or (self.keep_first > 0 and self.mask != "window"):
            raise ValueError("first positions are kept beside a sliding window only")
        if self.weighting == "sigmoid" and self.has_sinks:
            raise ValueError("a sink is a term of a softmax's sum: there is none under sigmoid weights")
        if self.score_cap < 0.0:
            raise ValueError(f"a cap of the scores is positive (or 0 for none), got {self.score_cap}")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are no multiple of {self.kv_heads} kv heads")
        if self.mask not in MASKS or (self.mask != "full") != (self.mask_size > 0):
            raise ValueError(f"mask {self.mask!r} of size {self.mask_size}: one of {MASKS}, the last two with a size > 0")
        if self.taps > ops.MAX_CONV_TAPS:
            raise ValueError(f"the convolution takes up to {ops.MAX_CONV_TAPS} taps, got {self.taps}")
        self.D = -(-max(self.d, self.dv) // 16) * 16
        if self.D > ops.MAX_PREPARED_HEAD:
            raise ValueError(f"head sizes up to {ops.MAX_PREPARED_HEAD}, got {self.d} and {self.dv}")
        pos = params.get("position")
        self.position = env.position_encoding(PartSpec(**pos) if isinstance(pos, dict) else pos) if pos else None
        self.rot = (self.position.rotary_dim or self.d) if self.position is not None else 0
        self.channels = (self.heads + self.kv_heads) * self.d + (0 if self.values == "keys" else self.kv_heads * self.dv)
        self.dtype, self.device = env.dtype, env.device
        # the mask as the attention kernels take it: > 0 a window, < 0 blocks of that many positions
        self.window = self.mask_size if self.mask == "window" else (-self.mask_size if self.mask == "chunk" else 0)
        self._w: dict = {}
        self.w_in = self.w_o = self.b_in = self.output_bias = self.conv_w = self.terms = self.weights = None

    # ---- weights
    def weight_specs(self):
        q, k, v = self.heads * self.d, self.kv_heads * self.d, self.kv_heads * self.dv
        own_values = self.values != "keys"
        specs = {"q": WeightSpec((q, self.hidden)), "k": WeightSpec((k, self.hidden)), "o": WeightSpec((self.hidden, self.heads * self.dv))}
        if own_values:
            specs["v"] = WeightSpec((v, self.hidden))
        if self.bias:
            specs.update({"q.b": WeightSpec((q,), role="vector"), "k.b": WeightSpec((k,), role="vector")})
            if own_values:
                specs["v.b"] = WeightSpec((v,), role="vector")
        if self.out_bias:
            specs["o.b"] = WeightSpec((self.hidden,), role="vector")
        if self.has_conv:
            specs.update({f"{n}.conv": WeightSpec((c, self.taps), role="vector") for n, c in (("q", q), ("k", k), ("v", v))[:3 if own_values else 2]})
        if self.weighting == "sigmoid":
            specs["pb"] = WeightSpec((self.heads,), role="vector")
        if self.has_sinks:
            specs["sink"] = WeightSpec((self.heads,), role="vector")
        if self.head_gate:
            specs["g"] = WeightSpec((self.heads, self.hidden))
        return specs

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def finalize(self):
        w = self._w
        qkv = ("q", "k", "v") if self.values != "keys" else ("q", "k")
        self.w_in = Weight(torch.cat([w.pop(n) for n in qkv + (("g",) if self.head_gate else ())], dim=0).contiguous())
        self.w_o = Weight(w.pop("o"))
        if self.bias:
            self.b_in = torch.cat([w.pop(n + ".b") for n in qkv]).contiguous()
        if self.out_bias:
            self.output_bias = w.pop("o.b")           # added by whoever norms the mixer's float output (the block's kernel), or by the product
        if self.has_conv:
            self.conv_w = torch.cat([w.pop(n + ".conv") for n in qkv], dim=0).contiguous()
        if self.keep_first or self.weighting == "sigmoid":
            self.weights = ops.KeyWeights(self.keep_first, self.weighting == "sigmoid", w.pop("pb") if self.weighting == "sigmoid" else None)
        terms = ops.ScoreTerms(self.score_cap, None, w.pop("sink") if self.has_sinks else None)
        self.terms = terms if terms.any() else None

    # ---- what it keeps
    def cache_spec(self):
        G, D = self.kv_heads, self.D
        return CacheSpec(self.mask, (PageTensor("k", (G, BLOCK, D)), PageTensor("v", (G, D, BLOCK))), self.mask_size, self.keep_first)

    def state_spec(self):
        return StateSpec(((self.taps - 1) * self.channels,), torch.float32) if self.taps > 1 else None

    def graph_step_arrays(self, layout):
        """The prompt kernel's work list (pairs of sequence and tile, most keys first) for a replayed step."""
        group, first = self.heads // self.kv_heads, layout.num_single_rows
        pairs = ops.prompt_tiles_capacity(layout.num_portions, layout.portion_tokens, group)
        return {("prompt_tiles", first, group): (2 * pairs, lambda q_lens, k_lens: ops.prompt_tiles(q_lens, k_lens, first, group, pairs))}

    # ---- compute
    def forward(self, h, ctx, cache, state):
        H, G, D = self.heads, self.kv_heads, self.D
        view = ctx.groups[cache.group]
        if not cache.writable:
            raise RuntimeError("this attention layer writes its own cache")
        proj = linear(h, self.w_in, out_dtype=torch.float32)
        pe = self.position
        k_pages, v_pages = cache["k"], cache["v"]
        q = ops.attn_prepare(proj, self.b_in, self.conv_w, state, ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs,
                             ctx.positions, pe.cos if pe is not None else None, pe.sin if pe is not None else None, self.rot,
                             bool(pe.interleaved) if pe is not None else False, self.eps, H, G, self.d, self.dv, D, self.dtype,
                             view.slot_mapping, k_pages, v_pages, qk_norm=self.qk_norm, values=self.values)
        o = ops.paged_attention(q, k_pages, v_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k, H, G, D, self.scale,
                                self.window, ctx, terms=self.terms, weights=self.weights)
        if self.head_gate or D != self.dv:
            o = ops.gate_heads(o, proj[:, self.channels:self.channels + H] if self.head_gate else None, H, self.dv, D)
        out_dtype = torch.float32 if getattr(ctx, "float_branch", False) else None
        if self.output_bias is not None and not getattr(ctx, "branch_bias_taken", False):
            return linear(o, self.w_o, out_dtype=out_dtype, bias=self.output_bias)
        return linear(o, self.w_o, out_dtype=out_dtype)


register_mixer("normed_attention", NormedAttention)
