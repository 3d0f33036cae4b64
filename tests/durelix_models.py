"""Small Durelix configurations for the tests, as ``config.json`` dictionaries. They differ from each other in every
size and constant: heads and groups (also one group per head, one head), key and value sizes that are no multiples of
anything and differ from each other, windows shorter than a page and none at all, convolutions of one to four taps
and none, rotations of part of a head, of a whole head and none, decays from one half to exactly one, dense and routed
feed-forwards in either order and a layer without one, routers with and without groups and identity experts, a model
without the second embedding table, a width that is no multiple of four."""

from __future__ import annotations


def left(heads, kv_heads, dim, vdim, scale, window=0, conv=0, rot=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        out["mask"] = {"size": window}
    if conv:
        out["conv"] = conv
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    return out


def right(heads, dim, vdim, decay, rot=None):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    return out


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=0, groups=None):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(l, r, mlp=None):
    return {"type": "parallel", "mixer": {"left": l, "right": r}, "mlp": mlp}


def model(vocab, width, layers, eps=1e-5, bigram=None):
    out = {"architecture": "Durelix", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if bigram:
        out["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return out


#: three layers of different geometry; windows of 20 and 7 tokens on pages of 8 or 16, one layer that sees everything
SMALL = model(97, 48, [
    layer(left(4, 2, 24, 16, 0.35, window=20, conv=3, rot=(10000.0, 16)), right(2, 16, 24, (0.9, 0.99), rot=(500.0, 8)),
          moe(6, 2, 20, identity=2, groups=(4, 2))),
    layer(left(3, 3, 40, 8, 0.2), right(1, 70, 70, (0.97,))),
    layer(left(2, 1, 12, 36, 0.5, window=7, conv=2, rot=(300.0, 12)), right(3, 8, 10, (1.0, 0.5, 0.999), rot=(50.0, 8)),
          dense(33)),
], eps=1e-5, bigram=(13, 31, 5))

#: one layer, sizes of one: a single head everywhere, a window of one token, one tap, one expert, one bucket
ONES = model(31, 20, [
    layer(left(1, 1, 6, 3, 1.1, window=1, conv=1, rot=(7.0, 2)), right(1, 4, 5, (0.8,), rot=(3.0, 4)), moe(1, 1, 7)),
], eps=1e-3, bigram=(1, 1, 1))

#: eight query heads on two groups, key heads beyond 128 elements, a router of three groups of which one is kept, no
#: second embedding table
WIDE = model(64, 64, [
    layer(left(8, 2, 32, 32, 0.3, window=33, conv=4, rot=(30000.0, 32)), right(2, 32, 96, (0.95, 0.999), rot=(2e5, 16)),
          moe(9, 4, 24, identity=3, groups=(3, 1))),
    layer(left(2, 2, 136, 20, 0.1, window=18, conv=4, rot=(1000.0, 64)), right(2, 130, 16, (0.9, 0.99), rot=(100.0, 130)),
          dense(64)),
], eps=1e-6)

#: a width and sizes that are multiples of nothing, the dense feed-forward first, three identity experts of five
ODD = model(53, 50, [
    layer(left(3, 1, 10, 14, 0.4, window=9, conv=2, rot=(100.0, 6)), right(2, 6, 9, (0.75, 0.98), rot=(40.0, 2)), dense(27)),
    layer(left(2, 2, 18, 5, 0.25, window=30, conv=3), right(1, 11, 13, (0.995,), rot=(9.0, 10)),
          moe(2, 2, 9, identity=3)),
], eps=1e-4, bigram=(7, 3, 11))


def routed_last(raw):
    """The same layers with the routed ones behind the others: a 16-bit run sends a token whose two experts nearly tie
    to another expert than the exact run does, a step and not a rounding, which in a last layer spoils that token's
    logits alone and in an earlier one those of every later token as well."""
    out = dict(raw)
    out["layers"] = sorted(raw["layers"], key=lambda l: bool(l["mlp"]) and l["mlp"]["kind"] == "moe")
    return out
