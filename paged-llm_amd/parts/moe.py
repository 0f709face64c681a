"""A feed-forward of routed experts: each token passes through ``top`` of ``experts`` small gated feed-forwards,
down(act(gate h) * (up h)) without biases, and the results are summed with router scores as weights.

Router: z = W_router h in float, scores s = softmax(z) over all router outputs.  The choice looks at s + correction (a
stored vector): the experts are cut into ``groups`` equal groups of neighbours, a group's mark is its largest corrected
score, and only experts of the ``keep`` best groups can be chosen; the ``top`` largest corrected scores among those win.
The weights are the chosen experts' scores s themselves (no renormalisation).  The last ``identity`` router outputs
stand for experts without weights that hand the token's own row back.

Options: ``scoring`` "sigmoid" scores every router output on its own, s = sigmoid(z); ``weight_on`` "input" lets the
weight multiply what the expert reads instead of what it returns, sum of expert(s h) (the factor goes onto the float sums of
the expert's first products, which are linear in the row); ``shared`` adds a gated feed-forward of the same form that
every token passes, times sigmoid(w_sg . h), one number per token, when it has a gate of its own.

On the GPU the (token, choice) pairs are sorted by expert and the experts' products run over tiles of a run of
rows each (``ops.moe_*``): nothing is read back by the host, so the step can be replayed from a graph, and a pair's
result does not depend on what else is in the batch.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import FeedForward, name_under
from .linear import Weight, gated_linear, linear
from .norm import rows_of
from .registry import BuildEnv, register_feed_forward
from .spec import WeightSpec


class RoutedExperts(FeedForward):
    """params: ``experts``, ``identity`` (pass-through experts behind them, default 0), ``top``, ``groups`` and ``keep``
    (defaults 1 and 1), ``intermediate_size`` (of one expert), ``activation`` (default "silu"), ``correction`` (a stored
    vector is added to the scores for the choice; default True), ``scoring`` ("softmax" or "sigmoid"), ``weight_on``
    ("output" or "input"), ``shared`` (None, or {``intermediate_size``, ``gate``: whether a token's gate exists}).
    Tensors: ``e<i>.gate``, ``e<i>.up`` [ff, width], ``e<i>.down`` [width, ff], ``router`` [experts + identity, width],
    ``correction`` [experts + identity]; ``shared.gate``, ``shared.up``, ``shared.down`` and ``shared.sg`` [1, width]."""
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.experts, self.identity = int(params["experts"]), int(params.get("identity") or 0)
        self.top, self.groups, self.keep = int(params["top"]), int(params.get("groups") or 1), int(params.get("keep") or 1)
        self.inter = int(params["intermediate_size"])
        self.activation = params.get("activation", "silu")
        self.has_correction = bool(params.get("correction", True))
        self.scoring, self.weight_on = params.get("scoring", "softmax"), params.get("weight_on", "output")
        shared = params.get("shared") or None
        self.shared_inter = int(shared["intermediate_size"]) if shared else 0
        self.shared_gate = bool(shared.get("gate", False)) if shared else False
        if self.scoring not in ops.MOE_SCORINGS or self.weight_on not in ("output", "input"):
            raise ValueError(f"scoring {self.scoring!r} (one of {sorted(ops.MOE_SCORINGS)}), weight_on {self.weight_on!r} (output or input)")
        self.n = self.experts + self.identity
        if self.activation not in ops.ACTIVATIONS:
            raise NotImplementedError(f"expert activation {self.activation!r}: one of {sorted(ops.ACTIVATIONS)}")
        if self.experts <= 0 or self.experts > ops.MOE_MAX_EXPERTS or self.n % self.groups or not 0 < self.keep <= self.groups \
                or not 0 < self.top <= (self.n // self.groups) * self.keep:
            raise ValueError(f"{self.experts} experts + {self.identity} pass-through in {self.groups} groups, {self.keep} kept, {self.top} chosen")
        self.dtype, self.device = env.dtype, env.device
        self._w: dict = {}
        self.w_gate_up = self.w_down = self.router = self.correction = self.w_shared_gate_up = self.w_shared_down = None

    def weight_specs(self):
        specs = {"router": WeightSpec((self.n, self.hidden), role="vector")}
        if self.has_correction:
            specs["correction"] = WeightSpec((self.n,), role="vector")
        for e in range(self.experts):
            specs[f"e{e}.gate"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.up"] = WeightSpec((self.inter, self.hidden))
            specs[f"e{e}.down"] = WeightSpec((self.hidden, self.inter))
        if self.shared_inter:
            specs.update({"shared.gate": WeightSpec((self.shared_inter, self.hidden)), "shared.up": WeightSpec((self.shared_inter, self.hidden)),
                          "shared.down": WeightSpec((self.hidden, self.shared_inter))})
            if self.shared_gate:
                specs["shared.sg"] = WeightSpec((1, self.hidden), role="vector")
        return specs

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def finalize(self):
        w, E = self._w, self.experts
        self.router = w.pop("router")
        if self.shared_inter:
            if self.shared_gate:          # the token's gate is one more row of the router's product (no expert: it is handed back as it is)
                self.router = torch.cat([self.router, w.pop("shared.sg")], dim=0).contiguous()
            self.w_shared_gate_up = Weight(torch.cat([w.pop("shared.gate"), w.pop("shared.up")], dim=0).contiguous(), "gated")
            self.w_shared_down = Weight(w.pop("shared.down"))
        self.correction = w.pop("correction") if self.has_correction else None
        # one tensor per kind of matrix, the experts one behind the other: [experts, 2 ff, width] with [gate; up], [experts, width, ff]
        self.w_gate_up = torch.stack([torch.cat([w.pop(f"e{e}.gate"), w.pop(f"e{e}.up")], dim=0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([w.pop(f"e{e}.down") for e in range(E)]).contiguous()

    def forward(self, h, ctx):
        h = rows_of(h)
        inside = self.weight_on == "input"
        routed = ops.moe_route(h, self.router, self.correction, self.groups, self.keep, self.top, self.scoring, extra=1 if self.shared_gate else 0)
        ids, weights = routed[0], routed[1]
        rows = ops.moe_tile_rows(ids.numel(), self.experts, h.dtype, self.hidden, self.inter, h.stride(0))
        sorted_pair, row_of_pair, tiles = ops.moe_align(ids, self.experts, rows)
        act = ops.moe_expert_gemm(h, self.w_gate_up, tiles, sorted_pair, self.top, True, self.activation, tile_rows=rows,
                                  pair_scale=weights if inside else None)
        out = ops.moe_expert_gemm(act, self.w_down, tiles, sorted_pair, self.top, False, tile_rows=rows)
        shared = gate = None
        if self.shared_inter:
            shared = linear(gated_linear(h, self.w_shared_gate_up, self.activation), self.w_shared_down, out_dtype=torch.float32)
            gate = routed[2] if self.shared_gate else None
        if getattr(ctx, "float_branch", False) and getattr(ctx, "branch_sum_ok", False):
            # whoever takes the branch forms the sum in its kernel
            return ops.ChoiceSum(out, h, row_of_pair, weights, inside, shared, gate)
        y = ops.moe_combine(out, h, row_of_pair, weights, inside, shared, gate)
        if getattr(ctx, "float_branch", False):
            return y
        return y if self.dtype == torch.float32 else ops.round_rows(y)


register_feed_forward("routed_experts", RoutedExperts)
