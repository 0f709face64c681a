"""Operations on the residual stream between layers (family "stream_op").

``concat_projection``: x <- W [x ; x0], one product over the stream and the embedding's output side by side (W is
[width, 2 width], the stream's columns first).  The operands are the two rows in the compute type, the result is a
new float stream (the product's float sums, never rounded)."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import StreamOp
from .linear import Weight, linear
from .registry import BuildEnv, register_stream_op
from .spec import WeightSpec


class ConcatProjection(StreamOp):
    """params: ``tensor_name`` (the matrix's own name under the part's prefix; "" is the prefix itself)."""

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.tensor_name = params.get("tensor_name", "weight")
        self.dtype, self.device = env.dtype, env.device
        self.weight: Weight | None = None
        self._w = None

    def weight_specs(self):
        return {self.tensor_name: WeightSpec((self.hidden, 2 * self.hidden))}

    def assign(self, name, tensor):
        if name != self.tensor_name:
            raise KeyError(name)
        self._w = tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def finalize(self):
        if self._w is not None:
            self.weight, self._w = Weight(self._w), None

    def forward(self, x, x0, ctx):
        T, H = x.shape
        both = torch.empty((T, 2 * H), dtype=self.dtype, device=x.device)
        ops.place_rows(x, both[:, :H])
        ops.place_rows(x0, both[:, H:])
        return linear(both, self.weight, out_dtype=torch.float32)


register_stream_op("concat_projection", ConcatProjection)


class AddEmbedding(StreamOp):
    """x <- x + x0: the embedding's output added to the stream, in float and in place (x0 itself is never written to).  When
    the layer behind it norms with a norm that can follow a sum in its kernel (``ctx.next_entry_norm`` with ``sum_then``), that
    norm's rows of the new stream come from the same kernel and travel beside the stream in ``ctx.launch_cache``
    (``ENTRY_ROWS``: (stream, norm, rows)), where a block over a float stream looks for them."""
    ENTRY_ROWS = "stream_entry_rows"

    def __init__(self, params: dict, env: BuildEnv):
        pass

    def forward(self, x, x0, ctx):
        if x.dtype != torch.float32 or x0.dtype != torch.float32 or x0 is x:
            raise RuntimeError("the embedding's output is added to a float stream, and is a tensor of its own")
        norm = getattr(ctx, "next_entry_norm", None)
        if norm is not None and hasattr(norm, "sum_then"):
            ctx.launch_cache[self.ENTRY_ROWS] = (x, norm, norm.sum_then(x, x0))
        else:
            ops.stream_add(x, x0)
            ctx.launch_cache[self.ENTRY_ROWS] = None
        return x


register_stream_op("add_embedding", AddEmbedding)
