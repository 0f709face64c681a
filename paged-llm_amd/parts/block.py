"""Pre-norm residual block: x += mixer(norm1(x)); x += feed_forward(norm2(x))
(pagedllm/model/llama.py:174-185).

The residual stream travels as (x, delta) with delta not yet added, so each norm adds the
previous branch's output in its own kernel; the sum is formed in float and rounded once to the
stream's element type, which is what a plain add in that type gives.
"""

from __future__ import annotations

import torch

from .base import Block
from .registry import register_block


class PreNormBlock(Block):
    """params: the four roles' prefixes in tensor names (mixer_norm, mixer, feed_forward_norm, feed_forward)."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}

    def accepts_partial_delta(self):
        return bool(getattr(self.parts["mixer_norm"], "accepts_partial_sums", False))

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        # What a branch returns goes to a norm as its delta.  If that norm can add float partial sums itself, the branch
        # is told so (``ctx.partial_sums_ok``) and may end in a product whose ranges of the inner dimension nobody has
        # added yet; for the feed-forward's output the model says what the next consumer takes.
        after_block = bool(getattr(ctx, "partial_sums_ok", False))
        h = p["mixer_norm"].pending(x, delta)             # summed and normed by whoever consumes it first
        ctx.partial_sums_ok = bool(getattr(p["feed_forward_norm"], "accepts_partial_sums", False))
        a = p["mixer"].forward(h, ctx, cache, state)
        x = h.residual()
        h = p["feed_forward_norm"].pending(x, a)
        ctx.partial_sums_ok = after_block
        m = p["feed_forward"].forward(h, ctx)
        return h.residual(), m


register_block("prenorm", PreNormBlock)


class BranchNormBlock(Block):
    """A block that norms what its branches return, not what they read, over a residual stream kept in float:

        x <- x + norm(mixer(x));   x <- x + norm(feed_forward(x))        (the second line only with a feed-forward)

    The branches read the stream itself (rounded to the compute type where that is not float); each branch's last
    product leaves float rows (``ctx.float_branch``), the norm runs in float and the sum stays in float: the stream is
    never rounded.  The kernel that norms and adds also writes the new stream in the compute type, which is the next
    branch's operand; it travels beside the stream in ``ctx.launch_cache`` so that the next block finds it.

    params: the roles' prefixes in tensor names; ``feed_forward`` False for a layer with the mixer alone (its specs
    then name no feed-forward roles)."""
    ROLES = {"mixer": "mixer", "mixer_norm": "norm", "feed_forward": "feed_forward", "feed_forward_norm": "norm"}
    _ROWS = "float_stream_rows"

    def __init__(self, params: dict, env):
        self.has_feed_forward = bool(params.get("feed_forward", True))
        if not self.has_feed_forward:
            self.ROLES = {"mixer": "mixer", "mixer_norm": "norm"}
        super().__init__({k: v for k, v in params.items() if k in self.ROLES and isinstance(v, str)}, env)
        self.dtype = env.dtype

    def _rows(self, x, ctx):
        """The stream in the compute type: what the kernel before left, or rounded now."""
        if x.dtype == self.dtype:
            return x
        held = ctx.launch_cache.get(self._ROWS)
        if held is not None and held[0] is x:
            return held[1]
        from ..csrc import ops
        return ops.round_rows(x)

    def _add(self, norm, x, branch, ctx, want_rows=True):
        rows = norm.add_to(x, branch, want_rows)
        ctx.launch_cache[self._ROWS] = (x, rows) if rows is not None else None

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        if delta is not None:
            raise RuntimeError("a block over a float stream takes the stream with every sum done")
        if x.dtype != torch.float32:
            raise RuntimeError("this block keeps its residual stream in float32 (an embedding with float_stream)")
        ctx.partial_sums_ok, ctx.float_branch = False, True
        a = p["mixer"].forward(self._rows(x, ctx), ctx, cache, state)
        self._add(p["mixer_norm"], x, a, ctx)
        if self.has_feed_forward:
            m = p["feed_forward"].forward(self._rows(x, ctx), ctx)
            self._add(p["feed_forward_norm"], x, m, ctx)
        ctx.float_branch = False
        return x, None


register_block("branch_norm", BranchNormBlock)


class SandwichNormBlock(Block):
    """A block with a norm in front of and behind every branch, over a residual stream kept in float:

        x <- x + m * norm_b(mixer(norm_a(x)));   x <- x + m * norm_d(feed_forward(norm_c(x)))    (the second line only with a feed-forward)

    The branches' last products leave float rows (``ctx.float_branch``); one kernel norms them, adds them times m to the
    stream in place and computes, from the row it still holds, the rows that whoever reads the stream next wants: this
    block's next norm, or the first norm of the layer that follows (``ctx.next_entry_norm``, set by the model), which
    travel beside the stream in ``ctx.launch_cache``.  A branch may hand a bias of its last product to that kernel
    (``output_bias`` of the part) instead of adding it itself.

    params: ``residual_mult`` (m), ``feed_forward`` (False: the mixer alone), and the roles' prefixes in tensor names."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_out_norm": "norm",
             "feed_forward_norm": "norm", "feed_forward": "feed_forward", "feed_forward_out_norm": "norm"}
    _ROWS = "sandwich_rows"

    def __init__(self, params: dict, env):
        self.has_feed_forward = bool(params.get("feed_forward", True))
        if not self.has_feed_forward:
            self.ROLES = {r: f for r, f in self.ROLES.items() if not r.startswith("feed_forward")}
        super().__init__({k: v for k, v in params.items() if k in self.ROLES and isinstance(v, str)}, env)
        self.mult = float(params.get("residual_mult", 1.0))
        self.dtype = env.dtype

    def entry_norm(self):
        return self.parts["mixer_norm"]

    def _entry_rows(self, x, ctx):
        """norm_a(x) in the compute type: what the kernel that last wrote x left for this norm, or computed now."""
        norm = self.parts["mixer_norm"]
        held = ctx.launch_cache.get(self._ROWS)
        if held is not None and held[0] is x and held[1] is norm:
            return held[2]
        return norm.forward(x)

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        if delta is not None:
            raise RuntimeError("a block over a float stream takes the stream with every sum done")
        if x.dtype != torch.float32:
            raise RuntimeError("this block keeps its residual stream in float32 (an embedding with float_stream)")
        after = getattr(ctx, "next_entry_norm", None)
        ctx.partial_sums_ok, ctx.float_branch = False, True
        ctx.branch_bias_taken = True          # a bias of a branch's last product is added by the kernel that norms the branch
        a = p["mixer"].forward(self._entry_rows(x, ctx), ctx, cache, state)
        bias = getattr(p["mixer"], "output_bias", None)
        if self.has_feed_forward:
            h = p["mixer_out_norm"].add_to(x, a, self.mult, bias=bias, then=p["feed_forward_norm"])
            ctx.branch_sum_ok = True      # a feed-forward may hand over a sum that the norm's kernel forms (``ops.ChoiceSum``)
            m = p["feed_forward"].forward(h, ctx)
            ctx.branch_sum_ok = False
            a, bias, last = m, getattr(p["feed_forward"], "output_bias", None), p["feed_forward_out_norm"]
        else:
            last = p["mixer_out_norm"]
        rows = last.add_to(x, a, self.mult, bias=bias, then=after, want_rows=after is not None)
        ctx.launch_cache[self._ROWS] = (x, after, rows) if after is not None else None
        ctx.float_branch = ctx.branch_bias_taken = False
        return x, None


register_block("sandwich_norm", SandwichNormBlock)


class FloatPreNormBlock(Block):
    """The pre-norm block over a residual stream kept in float:

        x <- x + mixer(norm_a(x));   x <- x + feed_forward(norm_b(x))        (the second line only with a feed-forward)

    The branches' last products leave float rows (``ctx.float_branch``); the kernel that adds them to the stream in place
    also computes, from the sums it holds, the rows of the norm that reads the stream next: this block's second norm, or
    the first norm of the layer that follows (``ctx.next_entry_norm``, set by the model), which travel beside the stream in
    ``ctx.launch_cache``.  The stream itself is never rounded.  The norms are of a kind with ``sum_then(stream, branch)``
    (a norm whose rows need nothing but the row's own elements, or that computes its statistics in that kernel).

    params: ``feed_forward`` (False: the mixer alone; the specs then name no feed-forward roles) and the roles' prefixes in
    tensor names."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}
    _ROWS = "float_prenorm_rows"

    def __init__(self, params: dict, env):
        self.has_feed_forward = bool(params.get("feed_forward", True))
        if not self.has_feed_forward:
            self.ROLES = {r: f for r, f in self.ROLES.items() if not r.startswith("feed_forward")}
        super().__init__({k: v for k, v in params.items() if k in self.ROLES and isinstance(v, str)}, env)
        self.dtype = env.dtype

    def build_parts(self, specs, env):
        super().build_parts(specs, env)
        for role, family in self.ROLES.items():
            if family == "norm" and not hasattr(self.parts[role], "sum_then"):
                raise ValueError(f"the norm {type(self.parts[role]).__name__} of role {role!r} cannot follow a sum in its kernel (no sum_then)")

    def entry_norm(self):
        return self.parts["mixer_norm"]

    def _entry_rows(self, x, ctx):
        """norm_a(x) in the compute type: what the kernel that last wrote x left for this norm, or computed now."""
        norm = self.parts["mixer_norm"]
        for key in (self._ROWS, "stream_entry_rows"):        # (the second: left by a stream operation in front of this layer)
            held = ctx.launch_cache.get(key)
            if held is not None and held[0] is x and held[1] is norm:
                ctx.launch_cache[key] = None
                return held[2]
        return norm.forward(x)

    def forward(self, x, delta, ctx, cache, state):
        p = self.parts
        if delta is not None:
            raise RuntimeError("a block over a float stream takes the stream with every sum done")
        if x.dtype != torch.float32:
            raise RuntimeError("this block keeps its residual stream in float32 (an embedding with float_stream)")
        after = getattr(ctx, "next_entry_norm", None)
        after = after if hasattr(after, "sum_then") else None
        ctx.partial_sums_ok, ctx.float_branch = False, True
        # a mixer made of two may hand over their weighted sum unformed (``ops.WeightedPair``) when the kernel behind it forms it
        reader = p["feed_forward_norm"] if self.has_feed_forward else after
        ctx.branch_pair_ok = bool(getattr(reader, "takes_weighted_pair", False))
        a = p["mixer"].forward(self._entry_rows(x, ctx), ctx, cache, state)
        ctx.branch_pair_ok = False
        if self.has_feed_forward:
            h = p["feed_forward_norm"].sum_then(x, a)
            ctx.branch_sum_ok = True      # a feed-forward may hand over a sum that the kernel behind it forms (``ops.ChoiceSum``)
            a = p["feed_forward"].forward(h, ctx)
            ctx.branch_sum_ok = False
        if after is not None:
            rows = after.sum_then(x, a)
            ctx.launch_cache[self._ROWS] = (x, after, rows)
        else:
            from ..csrc import ops
            ops.stream_add(x, a)                                # the sum alone: whoever reads the stream next norms for itself
            ctx.launch_cache[self._ROWS] = None
        ctx.float_branch = False
        return x, None


register_block("prenorm_float_stream", FloatPreNormBlock)
