"""Nesezen: a pre-norm decoder over a residual stream kept in float, x <- x + mixer(N(x)), x <- x + ff(N(x)), whose norm
computes no statistics (N(x) = tanh(alpha x) * w + b with a stored scalar alpha).  A layer holds one of three mixers and a
dense gated feed-forward, routed experts with a shared one, or no feed-forward; a layer may run with another layer's
weights (``weights_of``) and a cache or state of its own.

* ``attention``: grouped heads whose keys and values may differ in width, rotary pairs (i, i + r/2) on the first r
  elements of a head with the frequencies rescaled by wavelength, scores capped by c tanh(s / c), a sliding window.
* ``mlstm``: a matrix memory per head with exponential input gates under a running maximum and a normaliser.
* ``latent_attention``: queries through a normed latent, keys and values expanded from one cached normed latent per
  token, no positions, full causal mask, a sigmoid gate per head on the output.

``config.json``: ``architecture`` "Nesezen", ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list of {``type``, ``mixer``
(the mixer's sizes and constants), ``mlp`` ({``kind``: "dense", ``ff``}, {``kind``: "moe", ``expert``: {``ff``}, ``router``:
{``experts``, ``top``}, ``shared``: {``ff``}} or null), optionally ``weights_of``}.  Layer i's tensors are
``l<i>.norm1[.b|.alpha]``, ``l<i>.mix.*``, ``l<i>.norm2[.b|.alpha]``, ``l<i>.mlp.*``; outside the layers ``embed``,
``final.norm[.b|.alpha]`` and ``head``.  Importing this module registers the architecture."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep

MIXER_TYPES = ("attention", "mlstm", "latent_attention")
MLP_KINDS = ("dense", "moe")


@dataclass
class NesezenLayer:
    type: str
    mixer: dict
    mlp: dict | None
    weights_of: int | None = None


@dataclass
class NesezenConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: list = field(default_factory=list)
    max_positions: int = 4096
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_json(cls, cfg: dict) -> "NesezenConfig":
        layers = [NesezenLayer(str(l["type"]), dict(l["mixer"]), (dict(l["mlp"]) if l.get("mlp") is not None else None),
                               (int(l["weights_of"]) if l.get("weights_of") is not None else None)) for l in cfg["layers"]]
        out = cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                  max_positions=int(cfg.get("max_positions", 4096)), torch_dtype=str(cfg.get("torch_dtype") or "bfloat16"))
        out.validate()
        return out

    def owner_of(self, i: int) -> int | None:
        """The layer whose tensors layer i runs with: itself, or where its ``weights_of`` leads (a borrowed layer may be
        named in turn); None where that leaves the list or never ends."""
        for _ in range(len(self.layers) + 1):
            if not 0 <= i < len(self.layers):
                return None
            if self.layers[i].weights_of is None:
                return i
            i = self.layers[i].weights_of
        return None

    def validate(self) -> None:
        problems = []
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            problems.append("vocab, width and the number of layers must be positive")
        for i, l in enumerate(self.layers):
            if l.type not in MIXER_TYPES:
                problems.append(f"layer {i}: mixer type {l.type!r} is none of {MIXER_TYPES}")
            if l.mlp is not None and l.mlp.get("kind") not in MLP_KINDS:
                problems.append(f"layer {i}: feed-forward kind {l.mlp.get('kind')!r} is none of {MLP_KINDS}")
            if l.weights_of is not None:
                owner = self.owner_of(i)
                if owner is None:
                    problems.append(f"layer {i}: weights_of leads to no layer with weights of its own")
                elif self.layers[owner].type != l.type:
                    problems.append(f"layer {i}: weights_of names a layer of another type")
        if problems:
            raise ValueError("bad Nesezen config: " + "; ".join(problems))


def _rotary(rot: dict, head_dim: int) -> dict | None:
    dims = int(rot.get("dims") or 0) if rot else 0
    if dims <= 0:
        return None
    scaling = rot.get("scaling")
    if scaling:
        scaling = {"rope_type": "llama3", "factor": float(scaling["factor"]), "low_freq_factor": float(scaling["low"]),
                   "high_freq_factor": float(scaling["high"]), "original_max_position_embeddings": scaling["original"]}
    return {"kind": "rotary", "params": {"head_dim": head_dim, "theta": float(rot["base"]), "rotary_dim": dims, "interleaved": False,
                                         "scaling": scaling or None, "exact_frequencies": True}}


def _mixer_spec(kind: str, m: dict, eps: float) -> PartSpec:
    if kind == "attention":
        size = int((m.get("mask") or {}).get("size") or 0)
        return PartSpec("normed_attention", {
            "heads": int(m["heads"]), "kv_heads": int(m.get("kv_heads") or m["heads"]), "key_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
            "scale": float(m["scale"]), "eps": eps, "qk_norm": False, "score_cap": float(m.get("softcap") or 0.0),
            "position": _rotary(m.get("rot"), int(m["dim"])), "mask": "window" if size > 0 else "full", "mask_size": size})
    if kind == "mlstm":
        return PartSpec("mlstm", {"heads": int(m["heads"]), "key_dim": int(m["dim"]), "head_dim": int(m["vdim"]),
                                  "gate_cap": float(m.get("gate_cap") or 0.0), "eps": eps})
    return PartSpec("latent_attention", {"heads": int(m["heads"]), "plain_dim": int(m["dim"]), "rot_dim": 0, "head_dim": int(m["vdim"]),
                                         "rank": int(m["kv_rank"]), "q_rank": int(m["q_rank"]), "scale": float(m["scale"]), "window": 0,
                                         "position": None, "eps": eps, "head_gate": True})


def _mlp_spec(mlp: dict) -> PartSpec:
    if mlp["kind"] == "dense":
        return PartSpec("gated_mlp", {"intermediate_size": int(mlp["ff"]), "activation": "silu",
                                      "tensor_names": {"gate": "gate", "up": "up", "down": "down"}})
    r, shared = mlp["router"], mlp.get("shared")
    return PartSpec("routed_experts", {"experts": int(r["experts"]), "top": int(r["top"]), "intermediate_size": int(mlp["expert"]["ff"]),
                                       "activation": "silu", "correction": False, "scoring": "sigmoid", "weight_on": "input",
                                       "shared": {"intermediate_size": int(shared["ff"]), "gate": True} if shared else None})


def build_spec(cfg: NesezenConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("dynamic_tanh", {"weight_name": "", "bias_name": "b", "alpha_name": "alpha"})
    layers, index_of, schedule = [], {}, []
    for i, l in enumerate(cfg.layers):
        if l.weights_of is None:
            parts = {"mixer_norm": norm, "mixer": _mixer_spec(l.type, l.mixer, eps)}
            names = {"mixer_norm": "norm1", "mixer": "mix", "feed_forward": l.mlp is not None}
            if l.mlp is not None:
                parts.update({"feed_forward_norm": norm, "feed_forward": _mlp_spec(l.mlp)})
                names.update({"feed_forward_norm": "norm2", "feed_forward": "mlp"})
            index_of[i] = len(layers)
            layers.append(LayerSpec(f"l{i}", PartSpec("prenorm_float_stream", names), parts))
    for i, l in enumerate(cfg.layers):
        schedule.append(ScheduleStep(index_of[cfg.owner_of(i)]))
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "float_stream": True, "tensor_name": ""}),
        layers=layers, final_norm=norm, head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "tied": False, "tensor_name": ""}),
        schedule=schedule, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_id=None, stored_dtype=cfg.torch_dtype)


register_architecture(Architecture("Nesezen", NesezenConfig.from_json, build_spec))
