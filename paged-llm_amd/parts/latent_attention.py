"""Causal attention whose keys and values are expanded from one cached latent vector per token.

One product gives every head's query [plain | rot] and the down-projection [rank | rot]; the first ``rank`` elements,
RMS-normed with a weight, are the latent c, the last ``rot`` one rotated key part that all heads share.  A head's key
is [W_uk c ; rotated part] and its value W_uv c, so only c and the rotated part are kept per token.  The kernels never
expand the cache: the query is carried into the latent space (qa = W_uk^T q_plain, one small product per head), the
softmax runs over (qa . c + q_rot . k_rot) * scale and weighs the latents themselves, and W_uv is applied to the weighted
latent of each head.  That is attention with ONE key/value head shared by all query heads, key row [c | rotated part],
value c: the pages hold the key rows (padded to a multiple of 16 elements) and, transposed inside the page, the latents
once more as values, in the layouts of ``paged_attention``, whose kernels (the matrix-core ones in bfloat16, the plain one
in float32) then serve this mixer as they serve the grouped-head attention.  Latents wider than those kernels take keep
the key rows alone and use a plain kernel of this mixer.  A window (the last ``window`` positions) makes the pages a
windowed group.

Options that a layer may have: no rotated part at all (``rot_dim`` 0: no positions enter the scores), queries that come
through a latent of their own (``q_rank``: c_q = RMS norm of W_dq h with a weight, the heads' queries W_uq c_q), and a gate
per head on the attention's output (``head_gate``: head h's values times sigmoid((W_g h)_h)).
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import BLOCK, CacheSpec, Mixer, PageTensor
from .linear import Weight, linear
from .norm import rows_of
from .registry import BuildEnv, register_mixer
from .spec import PartSpec, WeightSpec


class LatentAttention(Mixer):
    """params: ``heads``, ``plain_dim``, ``rot_dim`` (per head; 0: none), ``head_dim`` (of the values), ``rank``, ``scale``,
    ``window`` (0: none), ``position`` (the rotary spec of the rot part; None without one), ``eps`` (of the latents' norms),
    ``q_rank`` (0: queries straight from the input; only without a rotated part), ``head_gate``.
    Tensors ``q`` [heads (plain + rot), width] or, with ``q_rank``, ``dq`` [q_rank, width], ``dq.norm`` [q_rank] and ``uq``
    [heads plain, q_rank]; ``dkv`` [rank + rot, width], ``dkv.norm`` [rank], ``uk`` [heads plain, rank], ``uv`` [heads
    head_dim, rank], ``o`` [width, heads head_dim]; ``g`` [heads, width] with ``head_gate``."""
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.plain, self.rot = int(params["heads"]), int(params["plain_dim"]), int(params["rot_dim"])
        self.P, self.rank = int(params["head_dim"]), int(params["rank"])
        self.scale, self.window, self.eps = float(params["scale"]), int(params.get("window") or 0), float(params["eps"])
        self.q_rank, self.head_gate = int(params.get("q_rank") or 0), bool(params.get("head_gate"))
        if self.rank > ops.MAX_LATENT_RANK or self.rot > ops.MAX_LATENT_ROT or self.rot % 2 or self.rot < 0 or self.plain <= 0:
            raise ValueError(f"latent attention takes a rank up to {ops.MAX_LATENT_RANK}, an even rotated width up to "
                             f"{ops.MAX_LATENT_ROT} and a plain width of at least 1; got {self.rank}, {self.rot}, {self.plain}")
        if self.q_rank and self.rot:
            raise NotImplementedError("queries through a latent together with a rotated part: the rotation of the expanded queries is not built")
        pos = params.get("position")
        if bool(pos) != (self.rot > 0):
            raise ValueError(f"a rotated part of {self.rot} elements and the position encoding {pos!r} do not go together")
        self.position = env.position_encoding(PartSpec(**pos) if isinstance(pos, dict) else pos) if pos else None
        if self.position is not None and (self.position.rotary_dim or self.rot) != self.rot:
            raise ValueError(f"the rotated part of {self.rot} elements turns as a whole, not {self.position.rotary_dim} of it")
        self.dtype, self.device = env.dtype, env.device
        self.width = -(-(self.rank + self.rot) // 16) * 16            # of a key row in the pages
        self.paged = self.width <= ops.MAX_HEAD_DIM_GENERIC           # the paged attention kernels take it
        self._w: dict = {}
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.norm_w = self.w_uq = self.q_norm_w = self.w_g = None

    def weight_specs(self):
        H = self.heads
        specs = {"dkv": WeightSpec((self.rank + self.rot, self.hidden)),
                 "dkv.norm": WeightSpec((self.rank,), role="vector", init="ones"), "uk": WeightSpec((H * self.plain, self.rank)),
                 "uv": WeightSpec((H * self.P, self.rank)), "o": WeightSpec((self.hidden, H * self.P))}
        if self.q_rank:
            specs.update({"dq": WeightSpec((self.q_rank, self.hidden)), "dq.norm": WeightSpec((self.q_rank,), role="vector", init="ones"),
                          "uq": WeightSpec((H * self.plain, self.q_rank))})
        else:
            specs["q"] = WeightSpec((H * (self.plain + self.rot), self.hidden))
        if self.head_gate:
            specs["g"] = WeightSpec((H, self.hidden))
        return specs

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def finalize(self):
        w, H = self._w, self.heads
        if self.q_rank:
            # one product of the input for both latents and the gates, as float sums: [dq | dkv | g]
            self.w_in = Weight(torch.cat([w.pop("dq"), w.pop("dkv")] + ([w.pop("g")] if self.head_gate else []), dim=0).contiguous())
            self.w_uq, self.q_norm_w = Weight(w.pop("uq")), w.pop("dq.norm")
        else:
            self.w_in = Weight(torch.cat([w.pop("q"), w.pop("dkv")], dim=0).contiguous())
            self.w_g = Weight(w.pop("g")) if self.head_gate else None
        self.w_o = Weight(w.pop("o"))
        self.w_uk_t = w.pop("uk").view(H, self.plain, self.rank).transpose(1, 2).contiguous()     # [heads, rank, plain]: qa = W_uk^T q
        self.w_uv = w.pop("uv").view(H, self.P, self.rank).contiguous()
        self.norm_w = w.pop("dkv.norm")

    def cache_spec(self):
        kind = "window" if self.window > 0 else "full"
        tensors = (PageTensor("k", (1, BLOCK, self.width)),) + ((PageTensor("v", (1, self.width, BLOCK)),) if self.paged else ())
        return CacheSpec(kind, tensors, self.window)

    def graph_step_arrays(self, layout):
        """The prompt kernel's work list of the paged attention (all heads are one group) for a replayed step."""
        if not self.paged:
            return {}
        first, group = layout.num_single_rows, self.heads
        pairs = ops.prompt_tiles_capacity(layout.num_portions, layout.portion_tokens, group)
        return {("prompt_tiles", first, group): (2 * pairs, lambda q_lens, k_lens: ops.prompt_tiles(q_lens, k_lens, first, group, pairs))}

    def forward(self, h, ctx, cache, state):
        H, d, r, rank, width = self.heads, self.plain, self.rot, self.rank, self.width
        view = ctx.groups[cache.group]
        pe = self.position
        cos, sin, inter = (pe.cos, pe.sin, bool(pe.interleaved)) if pe is not None else (None, None, False)
        k_pages, v_pages = cache["k"], (cache["v"] if self.paged else None)
        slots = view.slot_mapping if cache.writable else None
        gate = None
        if self.q_rank:
            rows = linear(h, self.w_in, out_dtype=torch.float32)
            T = rows.shape[0]
            q = torch.empty((T, H, width), dtype=self.dtype, device=rows.device)
            cq = ops.latent_prepare(rows, self.q_rank, ctx.positions, cos, sin, self.norm_w, self.eps, slots, k_pages, v_pages, q, H, d, r, rank,
                                    inter, q_latent=(0, self.q_rank, self.q_norm_w))
            q_plain = linear(cq, self.w_uq).view(T, H, d)
            if self.head_gate:
                gate = rows[:, self.q_rank + rank + r:]
        else:
            if self.head_gate:
                h = rows_of(h)
                gate = linear(h, self.w_g, out_dtype=torch.float32)
            rows = linear(h, self.w_in)
            T = rows.shape[0]
            q = torch.empty((T, H, width), dtype=rows.dtype, device=rows.device)
            ops.latent_prepare(rows, H * (d + r), ctx.positions, cos, sin, self.norm_w, self.eps, slots, k_pages, v_pages, q, H, d, r, rank, inter)
            q_plain = rows[:, :H * (d + r)].unflatten(1, (H, d + r))[:, :, :d]
        ops.gemm_heads(q_plain, self.w_uk_t, out=q[:, :, :rank])
        if self.paged:
            mixed = ops.paged_attention(q.view(T, H * width), k_pages, v_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k,
                                        H, 1, width, self.scale, self.window, ctx).view(T, H, width)[:, :, :rank]
        else:
            mixed = ops.latent_attention(q, rank, r, k_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k, self.scale, self.window)
        values = ops.gemm_heads(mixed, self.w_uv).view(T, H * self.P)
        if gate is not None:
            values = ops.gate_heads(values, gate, H, self.P, self.P)
        return linear(values, self.w_o, out_dtype=torch.float32 if getattr(ctx, "float_branch", False) else None)


register_mixer("latent_attention", LatentAttention)
