"""A decoder put together from a ModelSpec: embedding -> the scheduled layers -> last norm on the
wanted rows -> head.  It knows parts and the run order, not architectures."""

from __future__ import annotations

import torch

from ..cache.kv_cache import CacheGroup
from ..parts import registry
from ..parts.base import name_under, tensor_name
from ..parts.registry import BuildEnv
from ..parts.spec import ModelSpec, WeightSpec


class DecoderModel:
    EMBEDDING_STATE = "embedding"       # key of the embedding's per-request state among the states of the schedule's steps

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device, max_positions: int | None = None):
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_positions = max(spec.max_positions, max_positions or 0)
        env = BuildEnv(spec.hidden_size, dtype, self.device, self.max_positions, shared={})
        self.env = env
        self.embedding = registry.build("embedding", spec.embedding, env)
        self.blocks = []
        for layer in spec.layers:
            block = registry.build("block", layer.block, env)
            block.build_parts(layer.parts, env)
            self.blocks.append(block)
        # operations on the stream between layers, which schedule steps name as their entry
        self.stream_ops = [registry.build("stream_op", op.part, env) for op in spec.stream_ops]
        self.final_norm = registry.build("norm", spec.final_norm, env)
        self.head = registry.build("head", spec.head, env)
        self._ready = False

    # ------------------------------------------------------------------ weights
    def weight_specs(self) -> dict[str, WeightSpec]:
        s = self.spec
        out = {tensor_name(s.embedding_name, n): w for n, w in self.embedding.weight_specs().items()}
        for layer, block in zip(s.layers, self.blocks):
            out.update({tensor_name(layer.name, n): w for n, w in block.weight_specs().items()})
        for op, part in zip(s.stream_ops, self.stream_ops):
            out.update({tensor_name(op.name, n): w for n, w in part.weight_specs().items()})
        out.update({tensor_name(s.final_norm_name, n): w for n, w in self.final_norm.weight_specs().items()})
        out.update({tensor_name(s.head_name, n): w for n, w in self.head.weight_specs().items()})
        return out

    def optional_weights(self) -> dict[str, tuple]:
        """Tensors a checkpoint may carry although the model does not need them (a tied head
        stored a second time): name -> shape."""
        if getattr(self.head, "tied", False):
            return {f"{self.spec.head_name}.weight": (self.spec.vocab_size, self.spec.hidden_size)}
        return {}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        s = self.spec
        outside = [(s.embedding_name, self.embedding), (s.final_norm_name, self.final_norm), (s.head_name, self.head)]
        for prefix, part in outside + [(op.name, part) for op, part in zip(s.stream_ops, self.stream_ops)]:
            own = name_under(prefix, name)
            if own is not None and own in part.weight_specs():
                return part.assign(own, tensor)
            if "/" + name in part.weight_specs():             # a tensor that the part names outside its prefix
                return part.assign("/" + name, tensor)
        for layer, block in zip(s.layers, self.blocks):
            own = name_under(layer.name, name)
            if own:
                return block.assign(own, tensor)
        raise KeyError(name)

    def finalize(self) -> None:
        self.embedding.finalize()
        for b in self.blocks:
            b.finalize()
        for op in self.stream_ops:
            op.finalize()
        self.final_norm.finalize()
        self.head.finalize()
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.table)
        self._ready = True

    # ------------------------------------------------------------------ what the cache manager must provide
    def cache_groups(self) -> dict[str, CacheGroup]:
        """Schedule steps that own pages, grouped by what their mixers keep per token."""
        groups: dict[str, CacheGroup] = {}
        for pos, step in enumerate(self.spec.schedule):
            if step.cache_from is not None:
                continue
            cs = self.blocks[step.layer].cache_spec()
            if cs is None:
                continue
            name = cs.group_name()
            groups.setdefault(name, CacheGroup(name, cs, [])).owners.append(pos)
        return groups

    def state_specs(self) -> dict[int, object]:
        """Schedule step -> StateSpec for mixers with per-request state of fixed size."""
        out = {}
        if getattr(self.embedding, "state_spec", None) is not None and self.embedding.state_spec() is not None:
            out[self.EMBEDDING_STATE] = self.embedding.state_spec()       # (an embedding that looks at the token before)
        for pos, step in enumerate(self.spec.schedule):
            ss = self.blocks[step.layer].state_spec()
            if ss is not None:
                out[pos] = ss
        return out

    def graph_capturable(self, prompts: bool = False) -> bool:
        """True when every layer's parts only launch kernels (no host reads of device data, no Python-side
        state): a decode step (``prompts``: also a step with prompt portions) can then be captured into a HIP graph."""
        flag = "graph_capturable_prompts" if prompts else "graph_capturable"
        return all(b.graph_capturable(prompts) for b in self.blocks) and all(getattr(op, flag, False) for op in self.stream_ops)

    def graph_step_arrays(self, layout) -> dict:
        """Host-made integer arrays the layers' parts need for a replayed step of that layout (equal keys are one array)."""
        out = {}
        for b in self.blocks:
            out.update(b.graph_step_arrays(layout))
        return out

    # ------------------------------------------------------------------ compute
    def forward(self, ctx, kv_storage, states: dict) -> torch.Tensor:
        """Float logits [n, vocab] at ctx.logits_index (empty tensor when nothing is wanted;
        the layers still run to fill the cache)."""
        assert self._ready, "weights not loaded"
        stateful_embedding = hasattr(self.embedding, "forward_step")
        x = (self.embedding.forward_step(ctx, states.get(self.EMBEDDING_STATE)) if stateful_embedding
             else self.embedding.forward(ctx.input_ids))
        delta = None
        schedule = self.spec.schedule
        # the embedding's output for the stream operations: a tensor of its own where the layers add to the stream in place
        x0 = None
        if self.stream_ops:
            if stateful_embedding:
                x0 = self.embedding.forward_step(ctx, states.get(self.EMBEDDING_STATE), again=True)
            else:
                x0 = self.embedding.forward(ctx.input_ids) if getattr(self.embedding, "float_stream", False) else x
        last_takes_partial = bool(getattr(self.final_norm, "accepts_partial_sums", False))
        for pos, step in enumerate(schedule):
            block = self.blocks[step.layer]
            if step.entry is not None and delta is not None:
                raise RuntimeError("a stream operation takes the stream with every sum done")
            # the norm that reads the stream next, for a block that can compute its rows while it forms the stream's last sum
            following = schedule[pos + 1] if pos + 1 < len(schedule) else None
            ctx.next_entry_norm = (self.blocks[following.layer].entry_norm() if following is not None and following.entry is None else None)
            if step.entry is not None:
                # the stream operation in front of this layer may norm for the layer in the kernel that forms its sum
                ctx.next_entry_norm, after_op = block.entry_norm(), ctx.next_entry_norm
                x = self.stream_ops[step.entry].forward(x, x0, ctx)
                ctx.next_entry_norm = after_op
            cache = None
            if block.cache_spec() is not None:
                owner = pos if step.cache_from is None else step.cache_from
                cache = kv_storage.for_step(owner, writable=step.cache_from is None)
            # whether the delta this block hands on may be float partial sums: what consumes it next says
            ctx.partial_sums_ok = (self.blocks[schedule[pos + 1].layer].accepts_partial_delta() if pos + 1 < len(schedule)
                                   else last_takes_partial)
            x, delta = block.forward(x, delta, ctx, cache, states.get(pos))
        ctx.partial_sums_ok = False
        n = ctx.logits_index.numel()
        if n == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        h = self.final_norm.pending(x, delta, ctx.logits_index, write_residual=False)
        return self.head.forward(h)
