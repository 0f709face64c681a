"""Renadra: a pre-norm decoder over a residual stream kept in float, x <- x + mixer(N1(x)), x <- x + ff(N2(x)), with RMS
norms (plain weights) and a SiLU-gated feed-forward in the layers that have one.  The embedding is the scaled token row
plus a row of a second table chosen by a hash of the token before and the token itself (the table's last row for a
sequence's first token).  A range of layers may run several times in a row with the same weights (a cache and state of
its own per pass); in front of every pass but the first the embedding's output is added to the stream.

* ``parallel``: two mixers on the same rows, added with a factor each.  Left: grouped heads with biases on q and k, no
  value product (a value head is its key head before the rotation), rotary pairs (i, i + r/2) on the first r elements
  with frequencies blended by pair index and tables times 0.1 ln(factor) + 1, scores capped by c tanh(s / c), a sliding
  window that also keeps the sequence's first positions, and no softmax: a visible key weighs sigmoid(score + a number
  per head).  Right: linear attention with a constant decay per head over SiLU-activated q, k, v, normed over all heads
  and gated by a sigmoid.
* ``attention``: grouped heads with biases on all four products, rotary pairs (2i, 2i + 1), values divided by their root
  mean square, a sliding window, softmax.
* ``hgrn2``: a linear recurrence whose forget gate, bounded below per channel, decays the state's rows and whose complement
  is the key.

``config.json``: ``architecture`` "Renadra", ``vocab``, ``width``, ``norm.eps``, ``embedding`` {``scale``, ``bigram``: {``buckets``,
``mul_prev``, ``mul_cur``}}, ``layers`` (a list of {``type``, ``mixer``, ``mlp``: {``kind``: "dense", ``ff``} or null}) and optionally
``loop`` {``start``, ``stop``, ``times``}.  Layer i's tensors are ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``; outside
the layers ``embed``, ``bigram``, ``final.norm`` and ``head``.  Importing this module registers the architecture."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep, StreamOpSpec

MIXER_TYPES = ("parallel", "attention", "hgrn2")


@dataclass
class RenadraLayer:
    type: str
    mixer: dict
    mlp: dict | None


@dataclass
class RenadraConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float = 1.0
    bigram: dict | None = None               # {"buckets", "mul_prev", "mul_cur"}
    layers: list = field(default_factory=list)
    loop: dict | None = None                 # {"start", "stop", "times"}
    max_positions: int = 4096
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_json(cls, cfg: dict) -> "RenadraConfig":
        layers = [RenadraLayer(str(l["type"]), dict(l["mixer"]), (dict(l["mlp"]) if l.get("mlp") is not None else None)) for l in cfg["layers"]]
        emb, loop = cfg.get("embedding") or {}, cfg.get("loop")
        bigram = emb.get("bigram")
        out = cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_eps=float(cfg["norm"]["eps"]),
                  embedding_scale=float(emb.get("scale") or 1.0),
                  bigram={k: int(bigram[k]) for k in ("buckets", "mul_prev", "mul_cur")} if bigram else None, layers=layers,
                  loop={k: int(loop[k]) for k in ("start", "stop", "times")} if loop else None,
                  max_positions=int(cfg.get("max_positions", 4096)), torch_dtype=str(cfg.get("torch_dtype") or "bfloat16"))
        out.validate()
        return out

    def validate(self) -> None:
        problems = []
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            problems.append("vocab, width and the number of layers must be positive")
        if self.bigram is not None and self.bigram["buckets"] <= 0:
            problems.append("a bigram table needs a positive number of buckets")
        for i, l in enumerate(self.layers):
            if l.type not in MIXER_TYPES:
                problems.append(f"layer {i}: mixer type {l.type!r} is none of {MIXER_TYPES}")
            if l.mlp is not None and l.mlp.get("kind") != "dense":
                problems.append(f"layer {i}: feed-forward kind {l.mlp.get('kind')!r} (dense only)")
        if self.loop is not None and not (0 <= self.loop["start"] < self.loop["stop"] <= len(self.layers) and self.loop["times"] >= 1):
            problems.append(f"loop {self.loop}: 0 <= start < stop <= {len(self.layers)} layers, times >= 1")
        if problems:
            raise ValueError("bad Renadra config: " + "; ".join(problems))

    def run_order(self) -> list:
        """[(layer, whether a pass of the repeated range other than the first starts here)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        order = [(i, False) for i in range(start)]
        for p in range(times):
            order += [(i, p > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]


def _rotary(rot: dict | None, head_dim: int, interleaved: bool) -> dict | None:
    dims = int(rot.get("dims") or 0) if rot else 0
    if dims <= 0:
        return None
    scaling = rot.get("scaling")
    if scaling:
        scaling = {"rope_type": "yarn", "factor": float(scaling["factor"]), "original": float(scaling["original"]),
                   "fast": float(scaling["fast"]), "slow": float(scaling["slow"])}
    return {"kind": "rotary", "params": {"head_dim": head_dim, "theta": float(rot["base"]), "rotary_dim": dims, "interleaved": interleaved,
                                         "scaling": scaling or None, "exact_frequencies": True}}


def _attention_spec(m: dict, eps: float, left: bool) -> PartSpec:
    mask = m.get("mask") or {}
    size = int(mask.get("size") or 0)
    params = {"heads": int(m["heads"]), "kv_heads": int(m.get("kv_heads") or m["heads"]), "key_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
              "scale": float(m["scale"]), "eps": eps, "qk_norm": False, "position": _rotary(m.get("rot"), int(m["dim"]), interleaved=not left),
              "mask": "window" if size > 0 else "full", "mask_size": size, "bias": True}
    if left:
        params.update({"output_bias": False, "values": "keys", "score_cap": float(m.get("softcap") or 0.0), "weighting": "sigmoid",
                       "keep_first": int(mask.get("keep_first") or 0) if size > 0 else 0})
    else:
        params.update({"output_bias": True, "values": "normed"})
    return PartSpec("normed_attention", params)


def _mixer_spec(kind: str, m: dict, eps: float) -> PartSpec:
    if kind == "attention":
        return _attention_spec(m, eps, left=False)
    if kind == "hgrn2":
        return PartSpec("hgrn2", {"heads": int(m["heads"]), "key_dim": int(m["dim"]), "head_dim": int(m["vdim"]), "eps": eps})
    left, right = m["left"], m["right"]
    lightning = PartSpec("lightning", {"heads": int(right["heads"]), "key_dim": int(right["dim"]), "head_dim": int(right["vdim"]),
                                       "decay": [float(d) for d in right["decay"]], "eps": eps})
    return PartSpec("parallel", {"left": _attention_spec(left, eps, left=True), "right": lightning,
                                 "left_scale": float(m.get("left_scale", 1.0)), "right_scale": float(m.get("right_scale", 1.0))})


def build_spec(cfg: RenadraConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("rmsnorm", {"eps": eps, "weight_name": ""})
    layers = []
    for i, l in enumerate(cfg.layers):
        parts = {"mixer_norm": norm, "mixer": _mixer_spec(l.type, l.mixer, eps)}
        names = {"mixer_norm": "norm1", "mixer": "mix", "feed_forward": l.mlp is not None}
        if l.mlp is not None:
            parts.update({"feed_forward_norm": norm,
                          "feed_forward": PartSpec("gated_mlp", {"intermediate_size": int(l.mlp["ff"]), "activation": "silu",
                                                                 "tensor_names": {"gate": "gate", "up": "up", "down": "down"}})})
            names.update({"feed_forward_norm": "norm2", "feed_forward": "mlp"})
        layers.append(LayerSpec(f"l{i}", PartSpec("prenorm_float_stream", names), parts))
    order = cfg.run_order()
    stream_ops = [StreamOpSpec("loop", PartSpec("add_embedding", {}))] if any(again for _, again in order) else []
    schedule = [ScheduleStep(i, entry=0 if again else None) for i, again in order]
    if cfg.bigram is not None:
        embedding = PartSpec("hashed_bigram_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "tensor_name": "",
                                                         "pairs_name": "/bigram", **cfg.bigram})
    else:
        embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "float_stream": True, "tensor_name": ""})
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embedding=embedding, layers=layers, final_norm=norm,
        head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "tied": False, "tensor_name": ""}),
        schedule=schedule, stream_ops=stream_ops, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_id=None, stored_dtype=cfg.torch_dtype)


register_architecture(Architecture("Renadra", RenadraConfig.from_json, build_spec))
