"""Small Nesezen configurations for the tests: sizes, layer orders and constants that differ from one another in every
field, and single-layer ones that show one mechanism alone."""

import copy


def attention(heads=4, kv_heads=2, dim=24, vdim=40, size=21, rot_dims=16, base=1e4, scale=0.3, softcap=20.0, scaling="default"):
    """The attention layer with grouped heads, a partial rotation with rescaled frequencies, capped scores and a window."""
    if scaling == "default":
        scaling = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48}
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "rot": rot, "scale": scale,
            "softcap": softcap}


def mlstm(heads=3, dim=20, vdim=24, gate_cap=10.0):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}


def latent(heads=4, dim=16, vdim=24, kv_rank=48, q_rank=40, scale=0.25):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}


def dense(ff=136):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=40, shared=56):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(kind, mixer, mlp=None, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def model(width, vocab, layers, eps=1e-5):
    return {"architecture": "Nesezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": copy.deepcopy(layers)}


# All three mixers, key and value sizes that differ, a partial rotation with the rescaling's three ranges, groups of
# heads on a key head, a window that is no multiple of a page, two chosen experts with a shared one, a layer without a
# feed-forward, and every layer once more with borrowed weights.
_A = [layer("attention", attention(), dense()),
      layer("mlstm", mlstm(), moe()),
      layer("latent_attention", latent(), None)]
NESE_A = model(96, 300, _A + [layer(l["type"], l["mixer"], l["mlp"], weights_of=i) for i, l in enumerate(_A)], eps=1e-5)

# Another order; as many key heads as heads; head sizes that fit no tile and a width that is no multiple of 4; a window of
# exactly one page; the whole head rotated without rescaling; no cap on the scores; a memory with more than 64 key rows
# and more than 64 value columns; one chosen expert without a shared one, and every expert chosen.
NESE_B = model(50, 77, [
    layer("latent_attention", latent(heads=5, dim=6, vdim=10, kv_rank=20, q_rank=12, scale=0.4), moe(experts=3, top=1, ff=34, shared=0)),
    layer("mlstm", mlstm(heads=2, dim=70, vdim=66, gate_cap=5.0), dense(ff=70)),
    layer("attention", attention(heads=3, kv_heads=3, dim=10, vdim=6, size=16, rot_dims=10, base=33.0, scale=0.5, softcap=0.0, scaling=None),
          moe(experts=4, top=4, ff=10, shared=18)),
], eps=1e-3)

# A window of one position (a query sees itself alone); head sizes beyond 64 and 128; a latent wider than the paged
# kernels take; one key head for eight heads; no rotation at all in one layer; one head; gates without a cap.
NESE_C = model(64, 131, [
    layer("attention", attention(heads=2, kv_heads=1, dim=80, vdim=144, size=1, rot_dims=40, base=100.0, scale=0.11, softcap=5.0)),
    layer("latent_attention", latent(heads=2, dim=24, vdim=16, kv_rank=272, q_rank=64, scale=0.2), dense(ff=64)),
    layer("attention", attention(heads=8, kv_heads=1, dim=16, vdim=16, size=40, rot_dims=0, scale=0.25, softcap=30.0, scaling=None),
          moe(experts=5, top=3, ff=24, shared=8)),
    layer("mlstm", mlstm(heads=1, dim=16, vdim=128, gate_cap=0.0), None),
], eps=1e-6)

# One mechanism each, over a width of 64.
ALONE = {
    "attention": model(64, 120, [layer("attention", attention(heads=4, kv_heads=2, dim=16, vdim=16, size=19, rot_dims=8, base=50.0, scale=0.25))]),
    "mlstm": model(64, 120, [layer("mlstm", mlstm(heads=2, dim=32, vdim=32, gate_cap=8.0))]),
    "latent": model(64, 120, [layer("latent_attention", latent(heads=2, dim=32, vdim=16, kv_rank=32, q_rank=24, scale=0.18))]),
    "dense": model(64, 120, [layer("attention", attention(heads=1, kv_heads=1, dim=16, vdim=16, size=1, rot_dims=0, scaling=None), dense(ff=96))]),
    "experts": model(64, 120, [layer("attention", attention(heads=1, kv_heads=1, dim=16, vdim=16, size=1, rot_dims=0, scaling=None),
                                     moe(experts=8, top=3, ff=48, shared=32))]),
}
