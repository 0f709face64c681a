"""Two mixers side by side: both read the same rows and their outputs are added with a factor each,

    out = left_scale * left(h) + right_scale * right(h).

Each side is any registered mixer with parameters of its own; its tensors lie under the side's prefix (``left.*``,
``right.*``).  One side at most keeps pages and one side at most keeps a state of fixed size per request (the layer's
cache and its state slot are handed to whichever side declared them), so attention beside a recurrence is served by
the cache manager and the state slots as each alone would be.  Under a block whose sum-and-norm kernel takes it
(``ctx.branch_pair_ok``) the weighted sum is handed on unformed (``ops.WeightedPair``) and that kernel forms it.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Mixer, name_under, tensor_name
from .registry import BuildEnv, build, register_mixer
from .spec import PartSpec


class ParallelMixer(Mixer):
    """params: ``left``, ``right`` (mixer specs: {"kind", "params"}), ``left_scale``, ``right_scale``, and optionally
    ``left_name`` / ``right_name`` (the sides' prefixes in tensor names; defaults "left" and "right")."""

    def __init__(self, params: dict, env: BuildEnv):
        def spec_of(s):
            return s if isinstance(s, PartSpec) else PartSpec(s["kind"], dict(s.get("params") or {}))
        self.sides = [(params.get("left_name", "left"), build("mixer", spec_of(params["left"]), env), float(params.get("left_scale", 1.0))),
                      (params.get("right_name", "right"), build("mixer", spec_of(params["right"]), env), float(params.get("right_scale", 1.0)))]
        if sum(m.cache_spec() is not None for _, m, _ in self.sides) > 1 or sum(m.state_spec() is not None for _, m, _ in self.sides) > 1:
            raise ValueError("of two mixers side by side one at most keeps pages and one at most keeps a state per request")
        self.graph_capturable = all(getattr(m, "graph_capturable", False) for _, m, _ in self.sides)
        self.graph_capturable_prompts = all(getattr(m, "graph_capturable_prompts", False) for _, m, _ in self.sides)

    def weight_specs(self):
        return {tensor_name(prefix, name): spec for prefix, m, _ in self.sides for name, spec in m.weight_specs().items()}

    def assign(self, name, tensor):
        for prefix, m, _ in self.sides:
            own = name_under(prefix, name)
            if own is not None and own in m.weight_specs():
                return m.assign(own, tensor)
        raise KeyError(name)

    def finalize(self):
        for _, m, _ in self.sides:
            m.finalize()

    def cache_spec(self):
        return next((m.cache_spec() for _, m, _ in self.sides if m.cache_spec() is not None), None)

    def state_spec(self):
        return next((m.state_spec() for _, m, _ in self.sides if m.state_spec() is not None), None)

    def graph_step_arrays(self, layout):
        out = {}
        for _, m, _ in self.sides:
            out.update(m.graph_step_arrays(layout))
        return out

    def forward(self, h, ctx, cache, state):
        outs = [m.forward(h, ctx, cache if m.cache_spec() is not None else None, state if m.state_spec() is not None else None)
                for _, m, _ in self.sides]
        if any(not isinstance(o, torch.Tensor) or o.dim() != 2 for o in outs):
            raise RuntimeError("mixers side by side return rows (no partial sums)")
        a, b = outs[0].contiguous(), outs[1].contiguous()
        if getattr(ctx, "branch_pair_ok", False) and a.dtype == torch.float32 and b.dtype == torch.float32:
            return ops.WeightedPair(a, self.sides[0][2], b, self.sides[1][2])        # formed by the kernel that adds it to the stream
        return ops.scaled_sum(a, self.sides[0][2], b, self.sides[1][2])


register_mixer("parallel", ParallelMixer)
