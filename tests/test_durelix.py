"""The Durelix design without a GPU: its configuration, its parts' manifest and caches, and the plain
implementation's mechanisms against properties that follow from their definitions."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import durelix_models as M
import plain_durelix as P
from pyre_amd.config.model import ConfigError
from pyre_amd.registry import config_from_dict

F = torch.float64


@pytest.mark.parametrize("raw", [M.SMALL, M.ONES, M.WIDE, M.ODD])
def test_configuration_round_trip_and_manifest(raw):
    from pyre_amd.parts.base import PagedCacheSpec, StateCacheSpec
    from pyre_amd.parts.model import LayeredModel
    from pyre_amd.registry import get_architecture

    cfg = config_from_dict(raw)
    assert config_from_dict(cfg.to_dict()) == cfg and cfg.architecture == "Durelix"
    model = LayeredModel(get_architecture(cfg.architecture).build(cfg))
    names = {s.name: s.shape for s in model.tensor_specs()}
    width = raw["width"]
    assert names["embed"] == (raw["vocab"], width) and names["final.norm"] == (width,) and "head" not in names
    big = (raw.get("embedding") or {}).get("bigram")
    assert ("bigram" in names) == bool(big) and (not big or names["bigram"] == (big["buckets"] + 1, width))
    kept = model.cache_specs()
    assert len(kept) == len(raw["layers"]) + (1 if big else 0)
    for i, layer in enumerate(raw["layers"]):
        a, r, p = layer["mixer"]["left"], layer["mixer"]["right"], f"l{i}"
        assert names[f"{p}.mix.left.q"] == (a["heads"] * a["dim"], width) and names[f"{p}.mix.left.k"] == (a["kv_heads"] * a["dim"], width)
        assert names[f"{p}.mix.left.g"] == (a["heads"] * a["vdim"], width) and names[f"{p}.mix.left.sink"] == (a["heads"],)
        assert names[f"{p}.mix.left.q.norm"] == (a["dim"],) and names[f"{p}.mix.left.out"] == (width,) == names[f"{p}.mix.right.out"]
        assert (f"{p}.mix.left.v.conv" in names) == bool(a.get("conv"))
        if a.get("conv"):
            assert names[f"{p}.mix.left.v.conv"] == (a["kv_heads"] * a["vdim"], a["conv"])
        assert names[f"{p}.mix.right.v"] == (r["heads"] * r["vdim"], width) == names[f"{p}.mix.right.g"]
        # pages of keys and values with the window, the convolution's last rows (more than one tap), the matrix state
        pages = [s for s in kept[i] if isinstance(s, PagedCacheSpec)]
        states = [s for s in kept[i] if isinstance(s, StateCacheSpec)]
        assert len(pages) == 1 and pages[0].window == (a.get("mask") or {}).get("size", 0)
        channels = (a["heads"] + a["kv_heads"]) * a["dim"] + a["kv_heads"] * a["vdim"]
        want = ([(a["conv"] - 1, channels)] if a.get("conv", 0) > 1 else []) + [(r["heads"], r["dim"], r["vdim"])]
        assert [s.shape for s in states] == want
        mlp = layer["mlp"]
        assert (f"{p}.norm2" in names) == (mlp is not None)
        if mlp and mlp["kind"] == "moe":
            total = mlp["router"]["experts"] + mlp["router"].get("identity", 0)
            assert names[f"{p}.mlp.router"] == (total, width) and names[f"{p}.mlp.correction"] == (total,)
            assert f"{p}.mlp.e{mlp['router']['experts'] - 1}.gate" in names and f"{p}.mlp.e{mlp['router']['experts']}.gate" not in names
        elif mlp:
            assert names[f"{p}.mlp.up"] == (mlp["ff"], width) and f"{p}.mlp.gate" not in names
    if big:
        assert [s.shape for s in kept[-1]] == [(1,)]


def test_configurations_that_are_refused():
    def broken(change):
        raw = copy.deepcopy(M.SMALL)
        change(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)

    broken(lambda r: r["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 3))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 15))
    broken(lambda r: r["layers"][0]["mixer"]["right"].__setitem__("decay", [0.9]))
    broken(lambda r: r["layers"][0]["mixer"]["right"].__setitem__("decay", [0.9, 1.5]))
    broken(lambda r: r["layers"][0]["mlp"]["router"]["groups"].__setitem__("count", 3))
    broken(lambda r: r["layers"][0]["mlp"]["router"].__setitem__("top", 5))
    broken(lambda r: r["layers"][0].__setitem__("type", "serial"))
    broken(lambda r: r["layers"][2]["mlp"].__setitem__("kind", "glu"))
    broken(lambda r: r["norm"].__setitem__("eps", 0.0))


# ----------------------------------------------------------------------------- the plain mechanisms


def test_short_convolution_is_causal_and_starts_from_zeros():
    g = torch.Generator().manual_seed(1)
    u, taps = torch.randn(9, 5, generator=g, dtype=F), torch.randn(5, 3, generator=g, dtype=F)
    y = P.short_conv(u, taps)
    assert torch.allclose(y[0], taps[:, 2] * u[0]) and torch.allclose(y[1], taps[:, 2] * u[1] + taps[:, 1] * u[0])
    assert torch.allclose(y[6], taps[:, 0] * u[4] + taps[:, 1] * u[5] + taps[:, 2] * u[6])
    other = u.clone()
    other[7] += 1.0
    assert torch.equal(P.short_conv(other, taps)[:7], y[:7])
    one = torch.ones(5, 1, dtype=F)
    assert torch.equal(P.short_conv(u, one), u)


@pytest.mark.parametrize("rotate", [P.rotate_neighbours, P.rotate_halves])
def test_rotations_depend_on_the_distance_alone(rotate):
    g = torch.Generator().manual_seed(2)
    q, k = torch.randn(1, 1, 10, generator=g, dtype=F), torch.randn(1, 1, 10, generator=g, dtype=F)

    def at(x, pos):
        return rotate(x.expand(pos + 1, 1, 10).clone(), 50.0, 6)[pos, 0]

    assert torch.allclose(at(q, 0), q[0, 0]) and torch.allclose(at(q, 7)[6:], q[0, 0, 6:])
    assert abs(float(at(q, 9) @ at(k, 4)) - float(at(q, 25) @ at(k, 20))) < 1e-12
    assert abs(float(at(q, 9) @ at(k, 4)) - float(at(q, 9) @ at(k, 5))) > 1e-3
    # which elements are partners
    e = torch.zeros(1, 1, 10, dtype=F)
    e[0, 0, 0] = 1.0
    moved = at(e, 1).nonzero().flatten().tolist()
    assert moved == ([0, 1] if rotate is P.rotate_neighbours else [0, 3])


def _attention_weights():
    g = torch.Generator().manual_seed(3)
    c = M.left(2, 1, 4, 3, 0.7, window=5, conv=2, rot=(30.0, 4))
    w = {f"a.{n}": torch.randn(rows, 6, generator=g, dtype=F) for n, rows in (("q", 8), ("k", 4), ("v", 3), ("g", 6))}
    w.update({"a.o": torch.randn(6, 6, generator=g, dtype=F), "a.q.norm": torch.ones(4, dtype=F), "a.k.norm": torch.ones(4, dtype=F),
              "a.sink": torch.tensor([0.3, -1.0], dtype=F)})
    w.update({f"a.{n}.conv": torch.randn(rows, 2, generator=g, dtype=F) for n, rows in (("q", 8), ("k", 4), ("v", 3))})
    return c, w, torch.randn(12, 6, generator=g, dtype=F)


def test_the_window_and_the_sink():
    c, w, h = _attention_weights()
    base = P.sink_attention(h, w, "a", c, 1e-6)
    # a token that the window has passed (and the convolution no longer reaches) changes nothing
    other = h.clone()
    other[3] += 1.0
    assert torch.allclose(P.sink_attention(other, w, "a", c, 1e-6)[9:], base[9:], atol=1e-12)
    assert not torch.allclose(P.sink_attention(other, w, "a", c, 1e-6)[8], base[8], atol=1e-6)  # token 4's key holds row 3
    # a sink far below every score is no sink; a sink far above them leaves nothing of the output
    w["a.sink"] = torch.tensor([-80.0, -80.0], dtype=F)
    plain = P.sink_attention(h, w, "a", c, 1e-6)
    assert not torch.allclose(plain, base, atol=1e-3)
    w["a.sink"] = torch.tensor([80.0, 80.0], dtype=F)
    assert float(P.sink_attention(h, w, "a", c, 1e-6).abs().max()) < 1e-20 * max(1.0, float(plain.abs().max())) + 1e-25


def test_retention_is_the_decayed_sum_over_earlier_tokens():
    g = torch.Generator().manual_seed(4)
    c = M.right(2, 4, 3, (0.5, 1.0), rot=(20.0, 2))
    w = {f"r.{n}": torch.randn(rows, 5, generator=g, dtype=F) for n, rows in (("q", 8), ("k", 8), ("v", 6), ("g", 6))}
    w["r.o"] = torch.eye(6, dtype=F)
    h = torch.randn(7, 5, generator=g, dtype=F)
    got = P.retention(h, w, "r", c, 1e-6)
    q = P.rotate_halves((h @ w["r.q"].T).view(7, 2, 4), 20.0, 2)
    k = P.rotate_halves((h @ w["r.k"].T).view(7, 2, 4), 20.0, 2) * 4 ** -0.5
    v = (h @ w["r.v"].T).view(7, 2, 3)
    o = torch.zeros(7, 2, 3, dtype=F)
    for a, decay in enumerate((0.5, 1.0)):
        for t in range(7):
            for s in range(t + 1):
                o[t, a] += decay ** (t - s) * (q[t, a] @ k[s, a]) * v[s, a]
    want = P.unit_rms(o, 1e-6).reshape(7, 6) * P.silu(h @ w["r.g"].T)
    assert torch.allclose(got, want, atol=1e-12)


def test_the_choice_of_experts():
    s = torch.tensor([0.05, 0.30, 0.10, 0.05, 0.20, 0.30], dtype=F)
    none = torch.zeros(6, dtype=F)
    assert P.choose(s, none, 2, 1, 1)[0] == [1, 5]                       # the lower index among equals first
    assert P.choose(s, none, 2, 3, 1)[0] == [1, 0]                       # groups (0,1) (2,3) (4,5): the first of the two best
    assert P.choose(s, none, 3, 3, 2)[0] == [1, 5, 4]
    # the correction moves the choice, not the weight; choice scores below zero still count
    corr = torch.tensor([-1.0, -1.0, -0.5, -0.6, -2.0, -2.0], dtype=F)
    chosen, gap = P.choose(s, corr, 2, 3, 1)
    assert chosen == [2, 3] and abs(gap - 0.3) < 1e-12                    # group 1 at -0.4 against group 0 at -0.7
    h = torch.randn(3, 4, dtype=F)
    w = {"m.router": torch.randn(6, 4, dtype=F), "m.correction": corr}
    c = {"router": {"experts": 4, "identity": 2, "top": 2, "groups": {"count": 3, "keep": 1}}}
    for t, picks in enumerate(P.route(h, w, "m", c)):
        scores = torch.softmax(w["m.router"] @ h[t], -1)
        assert all(abs(float(wt - scores[e])) < 1e-15 for e, wt in picks) and len(picks) == 2


def test_identity_experts_hand_the_row_back():
    g = torch.Generator().manual_seed(6)
    h = torch.randn(4, 5, generator=g, dtype=F)
    c = {"kind": "moe", "expert": {"ff": 3}, "router": {"experts": 1, "identity": 2, "top": 2}}
    w = {"m.router": torch.randn(3, 5, generator=g, dtype=F), "m.correction": torch.tensor([-9.0, 0.0, 0.0], dtype=F),
         "m.e0.gate": torch.randn(3, 5, generator=g, dtype=F), "m.e0.up": torch.randn(3, 5, generator=g, dtype=F),
         "m.e0.down": torch.randn(5, 3, generator=g, dtype=F)}
    s = torch.softmax(h @ w["m.router"].T, -1)
    assert torch.allclose(P.moe_ff(h, w, "m", c), (s[:, 1] + s[:, 2])[:, None] * h, atol=1e-14)


def test_the_second_embedding_table():
    cfg = {"embedding": {"bigram": {"buckets": 5, "mul_prev": 7, "mul_cur": 3}}}
    w = {"embed": torch.arange(40, dtype=F).view(10, 4), "bigram": 100.0 * torch.arange(24, dtype=F).view(6, 4)}
    x = P.embed(w, cfg, [9, 2, 2])
    assert torch.equal(x[0], w["embed"][9] + w["bigram"][5])
    assert torch.equal(x[1], w["embed"][2] + w["bigram"][(9 * 7 + 2 * 3) % 5]) and torch.equal(x[2], w["embed"][2] + w["bigram"][(2 * 7 + 2 * 3) % 5])
    assert torch.equal(P.embed(w, {}, [9, 2]), w["embed"][[9, 2]])


def test_a_layer_norms_what_its_sublayers_return():
    from pyre_amd.weights import model_tensor_specs, random_state

    cfg = config_from_dict(M.ODD)
    state = random_state(model_tensor_specs(cfg), 5, 0.2, 0.2, dtype="float32")
    w = {k: v.double() for k, v in state.items()}
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    _, hidden = P.forward(w, M.ODD, ids, return_hidden=True)
    x0 = P.embed(w, M.ODD, ids)
    x1 = x0 + P.rms_norm(P.parallel_mixer(x0, w, "l0.mix", M.ODD["layers"][0]["mixer"], 1e-4), w["l0.norm1"], 1e-4)
    x2 = x1 + P.rms_norm(P.dense_ff(x1, w, "l0.mlp"), w["l0.norm2"], 1e-4)
    assert torch.allclose(hidden[0], x2, atol=1e-12)
    assert math.isfinite(float(P.closest_call(w, M.ODD, ids).min()))
