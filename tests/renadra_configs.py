"""Small Renadra configurations for the tests: sizes, layer orders and constants that differ from one another in every
field, and single-layer ones that show one mechanism alone."""

import copy
import math


def left(heads=4, kv_heads=2, dim=24, size=21, keep_first=3, rot_dims=16, base=1e4, scale=0.3, softcap=15.0, scaling="default"):
    """The attention side of a parallel mixer: sigmoid weights, values = keys, a window that keeps the first positions."""
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.0}
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": size, "keep_first": keep_first}, "rot": rot,
            "scale": scale, "softcap": softcap}


def right(heads=3, dim=20, vdim=24, decay=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay or [math.exp(-1.0 / (2.0 + 3 * h)) for h in range(heads)]}


def parallel(l=None, r=None, left_scale=0.7, right_scale=1.2):
    return {"left": l or left(), "right": r or right(), "left_scale": left_scale, "right_scale": right_scale}


def attention(heads=4, kv_heads=2, dim=24, vdim=40, size=21, rot_dims=16, base=1e4, scale=0.3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "rot": {"base": base, "dims": rot_dims}, "scale": scale}


def hgrn2(heads=3, dim=20, vdim=24):
    return {"heads": heads, "dim": dim, "vdim": vdim}


def dense(ff=136):
    return {"kind": "dense", "ff": ff}


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(width, vocab, layers, eps=1e-5, scale=0.6, bigram=(61, 5, 3), loop=None):
    out = {"architecture": "Renadra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": scale, "bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}},
           "layers": copy.deepcopy(layers)}
    if loop:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# All three mixers; a repeated range in the middle that runs three times; key and value sizes that differ; partial
# rotations; groups of heads on a key head; windows that are no multiple of a page; kept positions within the first page.
RENA_A = model(96, 300, [layer("hgrn2", hgrn2(), dense()),
                         layer("parallel", parallel(), dense(72)),
                         layer("attention", attention(), None),
                         layer("hgrn2", hgrn2(heads=2, dim=16, vdim=40), dense(40))], eps=1e-5, loop=(1, 3, 3))

# Another order, no repeated range; as many key heads as heads; head sizes that fit no tile and a width that is no
# multiple of 4; a window of exactly one page; the whole head rotated, without rescaling; no cap; kept positions beyond a
# page; states of more than 64 rows and more than 64 columns; more buckets than tokens; an embedding scale of one.
RENA_B = model(50, 77, [
    layer("attention", attention(heads=3, kv_heads=3, dim=10, vdim=6, size=16, rot_dims=10, base=33.0, scale=0.5), dense(70)),
    layer("parallel", parallel(left(heads=3, kv_heads=3, dim=10, size=16, keep_first=20, rot_dims=10, base=33.0, scale=0.5, softcap=0.0, scaling=None),
                               right(heads=2, dim=70, vdim=66), left_scale=1.0, right_scale=0.4), None),
    layer("hgrn2", hgrn2(heads=1, dim=70, vdim=66), dense(34)),
], eps=1e-3, scale=1.0, bigram=(1009, 1, 7))

# A window of one position (a query sees itself and the kept positions); head sizes beyond 64 and 128; one key head for
# eight heads; no rotation at all in one layer; the whole model repeated twice; no kept positions in one layer.
RENA_C = model(64, 131, [
    layer("parallel", parallel(left(heads=2, kv_heads=1, dim=80, size=1, keep_first=2, rot_dims=40, base=100.0, scale=0.11, softcap=5.0),
                               right(heads=1, dim=16, vdim=128))),
    layer("attention", attention(heads=8, kv_heads=1, dim=16, vdim=144, size=40, rot_dims=0, scale=0.25), dense(64)),
    layer("parallel", parallel(left(heads=8, kv_heads=1, dim=16, size=40, keep_first=0, rot_dims=16, base=5e5, scale=0.25, softcap=30.0,
                                    scaling={"factor": 16.0, "original": 32, "fast": 4.0, "slow": 0.5}), right(heads=4, dim=8, vdim=8)), dense(24)),
], eps=1e-6, bigram=(7, 3, 2), loop=(0, 3, 2))

# One mechanism each, over a width of 64.
ALONE = {
    "left": model(64, 120, [layer("parallel", parallel(left(heads=4, kv_heads=2, dim=16, size=19, keep_first=4, rot_dims=8, base=50.0, scale=0.25),
                                                       right(heads=1, dim=8, vdim=8), left_scale=1.0, right_scale=0.0))]),
    "right": model(64, 120, [layer("parallel", parallel(left(heads=1, kv_heads=1, dim=16, size=1, keep_first=0, rot_dims=0, scaling=None),
                                                        right(heads=2, dim=32, vdim=32), left_scale=0.0, right_scale=1.0))]),
    "attention": model(64, 120, [layer("attention", attention(heads=4, kv_heads=2, dim=16, vdim=16, size=19, rot_dims=8, base=50.0, scale=0.25))]),
    "hgrn2": model(64, 120, [layer("hgrn2", hgrn2(heads=2, dim=32, vdim=32))]),
    "dense": model(64, 120, [layer("hgrn2", hgrn2(heads=1, dim=8, vdim=8), dense(96))]),
    "loop": model(64, 120, [layer("hgrn2", hgrn2(heads=1, dim=8, vdim=8), dense(32))], loop=(0, 1, 4)),
}
