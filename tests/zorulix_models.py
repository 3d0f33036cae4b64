"""Small Zorulix configurations for the tests, as ``config.json`` dictionaries. They differ from each other in every
size and constant: heads and groups (also one group per head, one head), key and value sizes that are no multiples of
anything and differ from each other, windows shorter than a page and none at all, rotations of part of a head, of a
whole head, stretched ones and none, recurrent branches with fewer query/key heads than value heads, convolutions of one
to five taps, mixtures with and without a shared expert, with all experts taken and with more experts than a wave has
lanes, layers without a feed-forward, layers that read an earlier layer's keys and values through a wider or a narrower
window than its own, a model without the token side input, a width that is no multiple of four."""

from __future__ import annotations


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def attn(heads, kv_heads, dim, vdim, scale, window=0, rot=None, kv_from=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        out["mask"] = {"size": window}
    if rot:
        out["rot"] = rot
    if kv_from is not None:
        out["kv_from"] = kv_from
    return out


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def moe(experts, top, ff, shared=0):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attention(m, mlp=None):
    return {"type": "attention", "mixer": m, "mlp": mlp}


def parallel(left, right, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def model(vocab, width, layers, eps=1e-5, scale=None, side=0):
    out = {"architecture": "Zorulix", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if scale is not None:
        out["embedding"] = {"scale": scale}
    if side:
        out["token_side"] = {"dim": side}
    return out


#: four layers; the third reads the first one's keys and values through a wider window than that layer's own, on pages
#: of 8 or 16; stretched frequencies whose blend begins and ends inside the head
SMALL = model(97, 48, [
    attention(attn(4, 2, 12, 10, 0.3, window=20, rot=rot(10000.0, 8)), moe(6, 2, 20, shared=12)),
    parallel(attn(4, 1, 16, 24, 0.25, window=27, rot=rot(3000.0, 16, (4.0, 64, 8.0, 0.5))), delta(4, 2, 8, 12, 3), 0.7, 1.2,
             moe(5, 3, 16)),
    attention(attn(4, 2, 12, 10, 0.4, window=33, rot=rot(10000.0, 8), kv_from=0)),
    parallel(attn(2, 2, 20, 6, 0.2, window=7, rot=rot(500.0, 12)), delta(3, 3, 10, 7, 2), 1.0, 0.5, moe(4, 1, 24, shared=8)),
], eps=1e-5, scale=3.0, side=6)

#: sizes of one: a single head everywhere, a window of one token, one tap, one expert, one side column
ONES = model(31, 20, [
    attention(attn(1, 1, 2, 3, 1.1, window=1, rot=rot(7.0, 2)), moe(1, 1, 7)),
    parallel(attn(1, 1, 4, 1, 0.9, window=1), delta(1, 1, 3, 5, 1), 1.0, 1.0, moe(2, 1, 5, shared=1)),
], eps=1e-3, scale=1.0, side=1)

#: key heads beyond 128 elements, more experts than a wave has lanes, value heads of the recurrent branch fed by one
#: query/key head, a layer reading keys through a narrower window than their owner's, no window at all
WIDE = model(64, 64, [
    attention(attn(8, 2, 32, 32, 0.2, rot=rot(30000.0, 32)), moe(70, 4, 8, shared=40)),
    parallel(attn(2, 2, 136, 20, 0.1, window=18, rot=rot(1000.0, 64, (8.0, 32, 4.0, 1.0))), delta(4, 1, 130, 16, 4), 0.5, 0.9,
             moe(9, 9, 12)),
    attention(attn(8, 2, 32, 32, 0.3, window=21, rot=rot(30000.0, 32), kv_from=0), moe(3, 2, 24)),
    parallel(attn(6, 3, 8, 144, 0.35, window=40), delta(2, 2, 32, 96, 5), 1.3, 0.4),
], eps=1e-6, scale=8.0, side=4)

#: a width and sizes that are multiples of nothing, no token side input, no factor on the embedding, the recurrent layer
#: first, a layer without a feed-forward in the middle
ODD = model(53, 50, [
    parallel(attn(3, 1, 10, 14, 0.4, window=9, rot=rot(100.0, 6)), delta(6, 2, 6, 9, 4), 0.8, 0.9, moe(7, 3, 9, shared=5)),
    attention(attn(3, 3, 14, 5, 0.25, window=30)),
    attention(attn(5, 1, 6, 11, 0.5, window=11, rot=rot(9.0, 6)), moe(2, 2, 9)),
], eps=1e-4)


#: the recurrent layer first, one owner of keys read by two later layers through a narrower and a wider window than its
#: own, with a parallel layer between them; rotation of part of a head everywhere; a key head of 16 and of 48 elements in
#: the recurrent branches (the sizes that their kernel takes a wave a column group for)
ORDER = model(80, 40, [
    parallel(attn(2, 1, 24, 12, 0.3, window=14, rot=rot(2000.0, 10, (2.5, 20, 3.0, 0.7))), delta(4, 2, 16, 8, 2), 1.1, 0.6, moe(4, 2, 12, shared=6)),
    attention(attn(6, 3, 10, 14, 0.35, window=16, rot=rot(700.0, 4)), moe(3, 1, 20)),
    attention(attn(6, 3, 10, 14, 0.5, window=9, rot=rot(700.0, 4), kv_from=1), moe(8, 3, 6, shared=10)),
    parallel(attn(3, 3, 8, 8, 0.45, rot=rot(90.0, 8)), delta(2, 2, 48, 20, 3), 0.9, 1.0),
    attention(attn(6, 3, 10, 14, 0.2, window=26, rot=rot(700.0, 4), kv_from=1), moe(5, 5, 8, shared=4)),
], eps=1e-5, scale=5.0, side=3)


def routed_last(raw):
    """The same layers with a feed-forward in the last one only: a 16-bit run sends a token whose two experts nearly tie
    to another expert than the exact run does, a step and not a rounding, which in a last layer spoils that token's
    logits alone and in an earlier one those of every later token as well."""
    out = dict(raw)
    layers = [dict(l) for l in raw["layers"]]
    for l in layers[:-1]:
        l["mlp"] = None
    if layers[-1]["mlp"] is None:
        layers[-1]["mlp"] = moe(4, 2, 16, shared=8)
    out["layers"] = layers
    return out
