"""Token embedding (a row gather, pagedllm/model/llama.py:197) and the output head
(logits = rows * table^T in float, pagedllm/model/llama.py:203-216; tied = the embedding table)."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Part
from .linear import Weight, linear
from .registry import BuildEnv, register_embedding, register_head
from .spec import WeightSpec


class TokenEmbedding(Part):
    """params: ``vocab_size``; ``scale`` (the gathered row is multiplied by it; default none); ``float_stream`` (the
    rows leave as float32 whatever the compute type: the start of a residual stream that is summed in float); ``tensor_name`` (the table's own
    name under the part's prefix, default "weight"; "" is the prefix itself)."""

    def __init__(self, params: dict, env: BuildEnv):
        self.vocab = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.scale = float(params.get("scale") or 1.0)
        self.float_stream = bool(params.get("float_stream", False))
        self.tensor_name = params.get("tensor_name", "weight")
        self.dtype, self.device = env.dtype, env.device
        self.table: torch.Tensor | None = None

    def weight_specs(self):
        return {self.tensor_name: WeightSpec((self.vocab, self.hidden), role="table")}

    def assign(self, name, tensor):
        if name != self.tensor_name:
            raise KeyError(name)
        self.table = tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        if self.float_stream:
            return ops.embed_scaled(ids, self.table, self.scale, want_rows=False)[0]
        if self.scale != 1.0:
            raise NotImplementedError("a scaled embedding leaves as a float stream (float_stream)")
        return ops.embed_gather(ids, self.table)


class HashedBigramEmbedding(Part):
    """A token embedding to which a row of a second table is added, chosen by a hash of the token before and the token
    itself:  x = table[token] * scale + pairs[(previous * mul_prev + token * mul_cur) mod buckets], and the second table's
    last row (number ``buckets``) for a sequence's first token.  The rows leave as float32 (the start of a residual stream
    summed in float).  The token before a step's first token is per-request state: one int32 per slot, left there by the
    step before (``state_spec``); a request at position 0 has none, whatever its slot holds.

    params: ``vocab_size``, ``scale``, ``buckets``, ``mul_prev``, ``mul_cur``; ``tensor_name`` (the token table's own name
    under the part's prefix; "" is the prefix itself) and ``pairs_name`` (the second table's; "/name" is a name outside the prefix)."""
    float_stream = True

    def __init__(self, params: dict, env: BuildEnv):
        self.vocab = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.scale = float(params.get("scale") or 1.0)
        self.buckets, self.mul_prev, self.mul_cur = int(params["buckets"]), int(params["mul_prev"]), int(params["mul_cur"])
        if self.buckets <= 0:
            raise ValueError(f"a bigram table needs a positive number of buckets, got {self.buckets}")
        # (a b) mod m = ((a mod m) b) mod m: multipliers of any size become numbers below the buckets, and the kernel's products stay small
        self.mul_prev, self.mul_cur = self.mul_prev % self.buckets, self.mul_cur % self.buckets
        self.tensor_name = params.get("tensor_name", "weight")
        self.pairs_name = params.get("pairs_name", "pairs")
        self.dtype, self.device = env.dtype, env.device
        self.table: torch.Tensor | None = None
        self.pairs: torch.Tensor | None = None
        self._rows = None            # the bigram rows of the step under way, for a second gather of the same step

    def weight_specs(self):
        return {self.tensor_name: WeightSpec((self.vocab, self.hidden), role="table"),
                self.pairs_name: WeightSpec((self.buckets + 1, self.hidden), role="table")}

    def assign(self, name, tensor):
        t = tensor.to(device=self.device, dtype=self.dtype).contiguous()
        if name == self.tensor_name:
            self.table = t
        elif name == self.pairs_name:
            self.pairs = t
        else:
            raise KeyError(name)

    def state_spec(self):
        from .base import StateSpec
        return StateSpec((1,), torch.int32)

    def forward_step(self, ctx, state: torch.Tensor, again: bool = False) -> torch.Tensor:
        """The step's rows; ``again``: once more for the same step (the state has moved already)."""
        if not again:
            self._rows = torch.empty_like(ctx.input_ids)
        return ops.embed_bigram(ctx.input_ids, self.table, self.pairs, self.scale, self.buckets, self.mul_prev, self.mul_cur, state,
                                ctx.state_slots, ctx.seq_starts, ctx.cu_seqlens_q, ctx.num_seqs, self._rows, move_state=not again)


class LMHead(Part):
    def __init__(self, params: dict, env: BuildEnv):
        self.vocab = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.tied = bool(params.get("tied", False))
        self.tensor_name = params.get("tensor_name", "weight")      # the matrix's own name under the prefix ("": the prefix)
        self.dtype, self.device = env.dtype, env.device
        self.weight: torch.Tensor | None = None
        self._matrix = None

    def weight_specs(self):
        return {} if self.tied else {self.tensor_name: WeightSpec((self.vocab, self.hidden))}

    def assign(self, name, tensor):
        if name != self.tensor_name or self.tied:
            raise KeyError(name)
        self.weight = tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def tie(self, table: torch.Tensor) -> None:
        self.weight = table
        self._matrix = None

    def finalize(self) -> None:
        self._matrix = None

    def forward(self, h) -> torch.Tensor:
        if self._matrix is None:                      # (the tiled copy for decode steps, made once the matrix is there)
            self._matrix = Weight(self.weight)
        return linear(h, self._matrix, out_dtype=torch.float32)


register_embedding("token_embedding", TokenEmbedding)
register_embedding("hashed_bigram_embedding", HashedBigramEmbedding)
register_head("lm_head", LMHead)
