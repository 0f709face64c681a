"""RMS norm: x * rsqrt(mean(x^2) + eps) * w in float, eps inside the root, plain weight
(pagedllm/model/llama.py:74-83).

A block hands its mixer and feed-forward a ``PendingNorm`` rather than normed rows: the residual
sum and the norm are then done inside the consumer's first matrix product when that product's
kernel can take them in (few rows, decoding), or by the norm kernel when ``rows()`` is asked for.
Either way the consumer sees the same rows, and the block reads the new residual afterwards.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Norm
from .registry import BuildEnv, register_norm
from .spec import WeightSpec


class PendingNorm:
    """rows = norm(x[row_index] + delta[row_index]), not computed yet.  ``delta``: rows like x, or the float partial sums
    [ranges, rows, hidden] of the product that made them, which the norm kernel adds in order."""

    def __init__(self, weight: torch.Tensor, eps: float, x: torch.Tensor, delta: torch.Tensor | None = None,
                 row_index: torch.Tensor | None = None, write_residual: bool = True):
        self.weight, self.eps = weight, eps
        self.x, self.delta, self.row_index = x, delta, row_index
        self.write_residual = write_residual and delta is not None
        self._rows: torch.Tensor | None = None
        self._summed = delta is None            # True once x holds x + delta

    # what consumers may ask without forcing the computation
    @property
    def num_rows(self) -> int:
        return self.row_index.numel() if self.row_index is not None else self.x.shape[0]

    @property
    def shape(self):
        return (self.num_rows, self.x.shape[1])

    @property
    def dtype(self):
        return self.x.dtype

    @property
    def device(self):
        return self.x.device

    def rows(self) -> torch.Tensor:
        """The normed rows as a tensor (computed once by the norm kernel)."""
        if self._rows is None:
            delta = None if self._summed else self.delta
            self._rows = ops.rmsnorm(self.x, self.weight, self.eps, delta, self.row_index, self.write_residual)
            if delta is not None and self.write_residual:
                self._summed = True
        return self._rows

    def fusable(self) -> bool:
        """Whether a consumer's kernel may still take the sum and the norm in (not once the rows exist, and not when the
        sum comes as float partial sums of a product, which only the norm kernel adds)."""
        return self._rows is None and (self._summed or self.delta is None or self.delta.dim() == 2)

    def fused_arguments(self) -> dict:
        """Arguments for a kernel that takes the sum and the norm in; call ``fused_done`` after it."""
        x_out = None
        if not self._summed and self.write_residual:
            x_out = torch.empty_like(self.x)
        return dict(delta=None if self._summed else self.delta, norm_weight=self.weight, eps=self.eps, x_out=x_out,
                    row_index=self.row_index)

    def fused_done(self, args: dict) -> None:
        if args["x_out"] is not None:
            self.x = args["x_out"]              # the kernel wrote the new residual there
            self._summed = True

    def residual(self) -> torch.Tensor:
        """x + delta, after whoever consumed the rows has run (forces the sum if nobody did)."""
        if not self._summed and self.write_residual:
            self.rows()
        return self.x


def rows_of(h) -> torch.Tensor:
    return h if isinstance(h, torch.Tensor) else h.rows()


class RMSNorm(Norm):
    # ``delta`` may be the float partial sums [ranges, rows, hidden] of a product cut along its inner dimension
    accepts_partial_sums = True

    def __init__(self, params: dict, env: BuildEnv):
        """params: ``eps``; ``size`` (default: the model's width); ``weight_name`` (the weight's own name under the part's
        prefix, default "weight"; "" is the prefix itself); ``unit_offset`` (the checkpoint stores w - 1: the factor
        applied is 1 + what is stored, formed in float when the weight arrives)."""
        self.eps = float(params["eps"])
        self.size = int(params.get("size", env.hidden_size))
        self.weight_name = params.get("weight_name", "weight")
        self.unit_offset = bool(params.get("unit_offset", False))
        self.dtype, self.device = env.dtype, env.device
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {self.weight_name: WeightSpec((self.size,), role="vector", init="zeros" if self.unit_offset else "ones")}

    def assign(self, name, tensor):
        if name != self.weight_name:
            raise KeyError(name)
        w = tensor.to(device=self.device, dtype=torch.float32)
        self.weight = (w + 1.0 if self.unit_offset else w).contiguous()

    def forward(self, x, row_index=None):
        if x.dtype == torch.float32 and self.dtype != torch.float32:        # rows of a float stream, normed into the compute type
            return ops.rms_sandwich(x, None, None, 0.0, self.eps, w_next=self.weight, out_dtype=self.dtype, row_index=row_index)
        return ops.rmsnorm(x, self.weight, self.eps, None, row_index)

    def add_to(self, stream: torch.Tensor, branch: torch.Tensor, mult: float = 1.0, bias: torch.Tensor | None = None,
               then: "RMSNorm | None" = None, out: torch.Tensor | None = None, want_rows: bool = True):
        """stream += mult * norm(branch + bias), in place and in float (a block that norms what its branches return).
        Returns the new stream's rows in the compute type for whoever reads them next, computed in the same kernel:
        normed by ``then`` (the reader's own norm), or as they are; into ``out`` when given; None unless ``want_rows``."""
        if then is not None and (then.eps != self.eps or then.size != self.size):
            raise ValueError("the norm behind the sum shares this norm's width and eps")
        return ops.rms_sandwich(stream, branch, self.weight, mult, self.eps, w_next=then.weight if then is not None else None,
                                out=out, out_dtype=self.dtype if want_rows and out is None else None, bias=bias)

    takes_weighted_pair = True          # ``sum_then`` forms a branch that is the weighted sum of two (``ops.WeightedPair``) in its kernel

    def sum_then(self, stream: torch.Tensor, branch) -> torch.Tensor:
        """stream += branch in place (float, the branch as it is); returns this norm's rows of the new stream in the compute
        type, from the same kernel (a pre-norm block over a float stream)."""
        if isinstance(branch, ops.ChoiceSum):
            branch = branch.rows()
        return ops.rms_sandwich(stream, branch, None, 1.0, self.eps, w_next=self.weight, out_dtype=self.dtype)      # (a ``WeightedPair`` is formed by the kernel)

    def add_norm(self, x, delta, row_index=None, write_residual=True):
        return ops.rmsnorm(x, self.weight, self.eps, delta, row_index, write_residual)

    def pending(self, x, delta=None, row_index=None, write_residual=True):
        if x.dtype == torch.float32 and self.dtype != torch.float32 and delta is None:
            return Norm.pending(self, x, None, row_index, write_residual)       # rows of a float stream: normed at once, into the compute type
        return PendingNorm(self.weight, self.eps, x, delta, row_index, write_residual)


register_norm("rmsnorm", RMSNorm)


class LayerNorm(Norm):
    """Layer norm with weight and bias, y = (v - mean) / sqrt(var + eps) * w + b with var the mean of the squared
    deviations, computed in float whatever the compute type.  Two uses: ``forward`` norms rows of a stream (the last
    norm in front of the head) and ``add_to`` norms a branch's output and adds it to a float residual stream in the same
    kernel (a block that norms what its branches return, not what they read).

    params: ``eps``; ``size`` (default: the model's width); ``weight_name`` / ``bias_name``: the tensors' own names
    under the part's prefix (defaults "weight" and "bias"; "" is the prefix itself)."""

    def __init__(self, params: dict, env: BuildEnv):
        self.eps = float(params["eps"])
        self.size = int(params.get("size", env.hidden_size))
        self.weight_name = params.get("weight_name", "weight")
        self.bias_name = params.get("bias_name", "bias")
        self.dtype, self.device = env.dtype, env.device
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def weight_specs(self):
        return {self.weight_name: WeightSpec((self.size,), role="vector", init="ones"),
                self.bias_name: WeightSpec((self.size,), role="vector", init="normal")}

    def assign(self, name, tensor):
        t = tensor.to(device=self.device, dtype=torch.float32).contiguous()
        if name == self.weight_name:
            self.weight = t
        elif name == self.bias_name:
            self.bias = t
        else:
            raise KeyError(name)

    def forward(self, x, row_index=None):
        """The normed rows in the compute type (x: float or compute-type rows)."""
        return ops.layernorm(x, self.weight, self.bias, self.eps, None, row_index, self.dtype)

    def add_to(self, stream: torch.Tensor, branch: torch.Tensor, want_rows: bool = True):
        """stream += norm(branch), in place and in float; returns the new stream rounded to the compute type when that
        is another type than the stream's and ``want_rows`` (the next product's operand), else None."""
        out_dtype = self.dtype if want_rows and self.dtype != stream.dtype else None
        return ops.layernorm(branch, self.weight, self.bias, self.eps, stream, None, out_dtype)


register_norm("layernorm", LayerNorm)


class DynamicTanh(Norm):
    """A norm that computes no mean and no variance: y = tanh(alpha x) * w + b element by element, with a stored scalar
    alpha, in float whatever the compute type.  ``forward`` gives the rows of a stream (float or compute-type rows) in
    the compute type; ``sum_then`` adds a branch's float rows to a float residual stream in place and gives this
    norm's rows of the new stream from the same kernel (a pre-norm block over a float stream: the kernel that forms a
    sum also norms it for whoever reads the stream next).

    params: ``size`` (default: the model's width); ``weight_name`` / ``bias_name`` / ``alpha_name``: the tensors' own
    names under the part's prefix (defaults "weight", "bias", "alpha"; "" is the prefix itself)."""

    def __init__(self, params: dict, env: BuildEnv):
        self.size = int(params.get("size", env.hidden_size))
        self.weight_name = params.get("weight_name", "weight")
        self.bias_name = params.get("bias_name", "bias")
        self.alpha_name = params.get("alpha_name", "alpha")
        self.dtype, self.device = env.dtype, env.device
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.alpha: float | None = None

    def weight_specs(self):
        return {self.weight_name: WeightSpec((self.size,), role="vector", init="ones"),
                self.bias_name: WeightSpec((self.size,), role="vector", init="normal"),
                self.alpha_name: WeightSpec((), role="vector", init="ones")}

    def assign(self, name, tensor):
        if name == self.alpha_name:
            self.alpha = float(tensor.to(torch.float32))        # a constant of the kernel from here on
            return
        t = tensor.to(device=self.device, dtype=torch.float32).contiguous()
        if name == self.weight_name:
            self.weight = t
        elif name == self.bias_name:
            self.bias = t
        else:
            raise KeyError(name)

    def forward(self, x, row_index=None):
        if x.dtype != torch.float32:
            x = x.float()
        return ops.dynamic_tanh(x, self.alpha, self.weight, self.bias, None, row_index, self.dtype)

    def sum_then(self, stream: torch.Tensor, branch: torch.Tensor) -> torch.Tensor:
        """stream += branch in place (float); returns this norm's rows of the new stream in the compute type."""
        return ops.dynamic_tanh(stream, self.alpha, self.weight, self.bias, branch, None, self.dtype)


register_norm("dynamic_tanh", DynamicTanh)
