"""Rotary position encoding: float tables of cos and sin per position.

inv_freq[i] = 1 / theta^(2i/r) over the r rotated elements of a head; optional "llama3" rescale of the
low frequencies, or a "yarn" rescale (frequencies blended by pair index, both tables times 0.1 ln(factor) + 1); angle[p, i] = p * inv_freq[i] in float (pagedllm/model/llama.py:86-128).  The tables
hold r/2 columns (the reference's cat[freqs, freqs] repeats them).  The rotation itself is done by the
mixer's kernel, fused with the cache write; this part says how: ``rotary_dim`` = r (default: the whole
head, as in the reference) and ``interleaved`` (pairs (2i, 2i+1) instead of the reference's (i, i + r/2)).
"""

from __future__ import annotations

import math

import torch

from .base import PositionEncoding
from .registry import BuildEnv, register_position_encoding


def llama3_rescale(inv_freq: torch.Tensor, factor: float, low_freq_factor: float, high_freq_factor: float,
                   original_max_position_embeddings: int) -> torch.Tensor:
    """Waves longer than orig/low are slowed by `factor`, shorter than orig/high stay, those in
    between are blended.  The formula is taken from pagedllm/model/llama.py:86-97 as it stands there
    (it is the published llama3 rule; there is one way to write it)."""
    wavelen = 2 * math.pi / inv_freq
    low_wl = original_max_position_embeddings / low_freq_factor
    high_wl = original_max_position_embeddings / high_freq_factor
    smooth = (original_max_position_embeddings / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    blended = (1 - smooth) * inv_freq / factor + smooth * inv_freq
    out = torch.where(wavelen > low_wl, inv_freq / factor, inv_freq)
    middle = (wavelen <= low_wl) & (wavelen >= high_wl)
    return torch.where(middle, blended, out)


def yarn_rescale(inv_freq: torch.Tensor, base: float, factor: float, original: float, fast: float, slow: float) -> torch.Tensor:
    """Frequencies blended by the index of their pair: with idx(t) = r ln(original / (2 pi t)) / (2 ln base) the (real) index
    of the pair that makes t turns over ``original`` positions, lo = max(floor(idx(fast)), 0), hi = min(ceil(idx(slow)), r - 1)
    and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at f_i / factor * ramp_i + f_i (1 - ramp_i):
    the pairs below lo as they are, those above hi slowed by the factor."""
    r = 2 * inv_freq.numel()

    def index_of(turns: float) -> float:
        return r * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), r - 1)
    ramp = ((torch.arange(inv_freq.numel(), dtype=inv_freq.dtype) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return inv_freq / factor * ramp + inv_freq * (1.0 - ramp)


class RotaryEncoding(PositionEncoding):
    def __init__(self, params: dict, env: BuildEnv):
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.scaling = params.get("scaling")
        self.rotary_dim = int(params.get("rotary_dim") or self.head_dim)
        self.interleaved = bool(params.get("interleaved", False))
        # True: every frequency theta^(-2i/r) is formed in double precision and rounded to float once (default: float
        # arithmetic all the way, as the reference's code has it; the two differ in the last place of some frequencies)
        self.exact_frequencies = bool(params.get("exact_frequencies", False))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary encoding turns pairs of elements: the rotated width must be even and at most the head "
                             f"size {self.head_dim}, got {self.rotary_dim}")
        if self.scaling:
            kind = self.scaling.get("rope_type", self.scaling.get("type"))
            if kind not in ("llama3", "yarn"):
                raise NotImplementedError(f"rope_type={kind!r} not supported (default, llama3 and yarn only)")
        self.device = env.device
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.num_positions = 0

    def _yarn(self) -> dict | None:
        s = self.scaling
        return s if s and s.get("rope_type", s.get("type")) == "yarn" else None

    def table_factor(self) -> float:
        """What both tables are multiplied by: 0.1 ln(factor) + 1 under the "yarn" rescaling, else 1."""
        s = self._yarn()
        return 0.1 * math.log(float(s["factor"])) + 1.0 if s else 1.0

    def inverse_frequencies(self) -> torch.Tensor:
        d = self.rotary_dim
        if self._yarn():
            # (always formed in double precision and rounded once)
            s = self._yarn()
            inv_freq = torch.tensor([self.theta ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
            return yarn_rescale(inv_freq, self.theta, float(s["factor"]), float(s["original"]), float(s["fast"]), float(s["slow"])).to(torch.float32)
        if self.exact_frequencies:
            inv_freq = torch.tensor([self.theta ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float64)
            if self.scaling:
                s = self.scaling
                inv_freq = llama3_rescale(inv_freq, float(s["factor"]), float(s.get("low_freq_factor", 1.0)), float(s.get("high_freq_factor", 4.0)),
                                          int(s.get("original_max_position_embeddings", 8192)))
            return inv_freq.to(torch.float32)
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        if self.scaling:
            s = self.scaling
            inv_freq = llama3_rescale(inv_freq, float(s["factor"]), float(s.get("low_freq_factor", 1.0)),
                                      float(s.get("high_freq_factor", 4.0)),
                                      int(s.get("original_max_position_embeddings", 8192)))
        return inv_freq

    def prepare(self, max_positions: int) -> None:
        if max_positions <= self.num_positions:
            return
        t = torch.arange(max_positions, dtype=torch.float32)
        angles = torch.outer(t, self.inverse_frequencies())          # [P, rotary_dim/2], float
        mag = self.table_factor()
        self.cos = (angles.cos() * mag if mag != 1.0 else angles.cos()).to(self.device).contiguous()
        self.sin = (angles.sin() * mag if mag != 1.0 else angles.sin()).to(self.device).contiguous()
        self.num_positions = max_positions


register_position_encoding("rotary", RotaryEncoding)
