"""The Zorulix design without a GPU: its configuration, its parts' manifest and caches, and the plain
implementation's mechanisms against properties that follow from their definitions."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_zorulix as P
import zorulix_models as M
from pyre_amd.config.model import ConfigError
from pyre_amd.registry import config_from_dict

F = torch.float64


@pytest.mark.parametrize("raw", [M.SMALL, M.ONES, M.WIDE, M.ODD, M.ORDER])
def test_configuration_round_trip_and_manifest(raw):
    from pyre_amd.parts.base import PagedCacheSpec, StateCacheSpec
    from pyre_amd.parts.model import LayeredModel
    from pyre_amd.registry import get_architecture

    cfg = config_from_dict(raw)
    assert config_from_dict(cfg.to_dict()) == cfg and cfg.architecture == "Zorulix"
    model = LayeredModel(get_architecture(cfg.architecture).build(cfg))
    names = {s.name: s.shape for s in model.tensor_specs()}
    width, side = raw["width"], (raw.get("token_side") or {}).get("dim", 0)
    assert names["embed"] == (raw["vocab"], width) == names["head"] and names["final.norm"] == (width,)
    assert ("side.embed" in names) == bool(side) and (not side or names["side.embed"] == (raw["vocab"], side * len(raw["layers"])))
    kept = model.cache_specs()
    assert len(kept) == len(raw["layers"])
    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}", layer["mixer"]
        assert (f"{p}.side.gate" in names) == bool(side)
        if side:
            assert names[f"{p}.side.gate"] == (side, width) and names[f"{p}.side.proj"] == (width, side) and names[f"{p}.side.norm"] == (width,)
        if layer["type"] == "attention":
            assert names[f"{p}.mix.q"] == (m["heads"] * m["dim"], width) == (names[f"{p}.mix.q.norm"][0], width)
            assert names[f"{p}.mix.q.b"] == (m["heads"] * m["dim"],) and names[f"{p}.mix.o"] == (width, m["heads"] * m["vdim"])
            own = "kv_from" not in m
            assert (f"{p}.mix.k" in names) == own == (f"{p}.mix.v.b" in names) == (f"{p}.mix.k.norm" in names) and f"{p}.mix.o.b" not in names
            if own:
                assert names[f"{p}.mix.k"] == (m["kv_heads"] * m["dim"], width) and names[f"{p}.mix.v"] == (m["kv_heads"] * m["vdim"], width)
                # pages are given back by the widest window among the layer and those that read its pages
                windows = [(m.get("mask") or {}).get("size", 0)] + [(l["mixer"].get("mask") or {}).get("size", 0)
                                                                     for l in raw["layers"] if l["mixer"].get("kv_from") == i]
                assert [type(s) for s in kept[i]] == [PagedCacheSpec] and kept[i][0].window == (0 if 0 in windows else max(windows))
            else:
                assert kept[i] == [] and model.schedule[i].cache_from == m["kv_from"]
        else:
            a, r = m["left"], m["right"]
            assert names[f"{p}.mix.left.k"] == (a["kv_heads"] * a["dim"], width) and names[f"{p}.mix.left.o.b"] == (width,)
            assert f"{p}.mix.left.q.norm" not in names and names[f"{p}.mix.left.v.b"] == (a["kv_heads"] * a["vdim"],)
            assert names[f"{p}.mix.right.q"] == (r["kv_heads"] * r["dim"], width) == names[f"{p}.mix.right.k"]
            assert names[f"{p}.mix.right.v"] == (r["heads"] * r["vdim"], width) and names[f"{p}.mix.right.b"] == (r["heads"], width)
            assert names[f"{p}.mix.right.v.conv"] == (r["heads"] * r["vdim"], r["conv"]) and names[f"{p}.mix.right.A_log"] == (r["heads"],)
            assert names[f"{p}.mix.right.a2"][0] == r["heads"] * r["dim"] == names[f"{p}.mix.right.dt_bias"][0]
            assert names[f"{p}.mix.right.g2"][0] == r["heads"] * r["vdim"] and names[f"{p}.mix.right.norm"] == (r["vdim"],)
            assert names[f"{p}.mix.right.a1"] == (None, width) and names[f"{p}.mix.right.o"] == (width, r["heads"] * r["vdim"])
            channels = 2 * r["kv_heads"] * r["dim"] + r["heads"] * r["vdim"]
            states = [s.shape for s in kept[i] if isinstance(s, StateCacheSpec)]
            assert states == [(r["heads"], r["vdim"], r["dim"])] + ([(r["conv"] - 1, channels)] if r["conv"] > 1 else [])
            assert [s.window for s in kept[i] if isinstance(s, PagedCacheSpec)] == [(a.get("mask") or {}).get("size", 0)]
        mlp = layer["mlp"]
        assert (f"{p}.norm2" in names) == (mlp is not None)
        if mlp:
            E = mlp["router"]["experts"]
            assert names[f"{p}.mlp.router"] == (E, width) and names[f"{p}.mlp.router.b"] == (E,)
            assert names[f"{p}.mlp.e{E - 1}.gate"] == (mlp["expert"]["ff"], width) and f"{p}.mlp.e{E}.gate" not in names
            assert (f"{p}.mlp.shared.sg" in names) == ("shared" in mlp)
            if "shared" in mlp:
                assert names[f"{p}.mlp.shared.down"] == (width, mlp["shared"]["ff"]) and names[f"{p}.mlp.shared.sg"] == (1, width)


def test_configurations_that_are_refused():
    def broken(change):
        raw = copy.deepcopy(M.SMALL)
        change(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)

    broken(lambda r: r["layers"][0]["mixer"].__setitem__("kv_heads", 3))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].__setitem__("dims", 7))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].__setitem__("dims", 14))
    broken(lambda r: r["layers"][1]["mixer"]["left"]["rot"]["scaling"].__setitem__("factor", 0.0))
    broken(lambda r: r["layers"][1]["mixer"]["right"].__setitem__("kv_heads", 3))
    broken(lambda r: r["layers"][1]["mixer"]["right"].__setitem__("conv", 0))
    broken(lambda r: r["layers"][1]["mixer"].pop("left_scale"))
    broken(lambda r: r["layers"][2]["mixer"].__setitem__("kv_from", 1))      # a parallel layer keeps no such keys
    broken(lambda r: r["layers"][2]["mixer"].__setitem__("kv_from", 2))      # itself
    broken(lambda r: r["layers"][2]["mixer"].__setitem__("dim", 8))          # other sizes than the owner's
    broken(lambda r: r["layers"][0]["mlp"]["router"].__setitem__("top", 7))
    broken(lambda r: r["layers"][0].__setitem__("type", "serial"))
    broken(lambda r: r["layers"][0]["mlp"].__setitem__("kind", "glu"))
    broken(lambda r: r["norm"].__setitem__("eps", 0.0))


def test_window_and_sink_of_the_plain_attention():
    g = torch.Generator().manual_seed(1)
    T, H, G, d, dv = 9, 4, 2, 5, 3
    q, k, v = (torch.randn(T, n, e, generator=g, dtype=F) for n, e in ((H, d), (G, d), (G, dv)))
    out = P.window_attention(q, k, v, 0.7, 4, True).reshape(T, H, dv)
    i, hd = 7, 3
    s = torch.stack([(q[i, hd] @ k[j, 1]) * 0.7 for j in range(4, 8)])
    want = (torch.exp(s) / (1.0 + torch.exp(s).sum())) @ v[4:8, 1]
    assert torch.allclose(out[i, hd], want, atol=1e-12)
    # without a sink the weights sum to one; a window of one token returns the token's own value
    plain = P.window_attention(q, k, v, 0.7, 1, False).reshape(T, H, dv)
    assert torch.allclose(plain[5, 0], v[5, 0], atol=1e-12) and torch.allclose(plain[5, 3], v[5, 1], atol=1e-12)
    # no window: the first query sees itself alone, and the sink takes its share
    everything = P.window_attention(q, k, v, 0.7, 0, True).reshape(T, H, dv)
    s0 = (q[0, 0] @ k[0, 0]) * 0.7
    assert torch.allclose(everything[0, 0], torch.exp(s0) / (1 + torch.exp(s0)) * v[0, 0], atol=1e-12)


def test_rotation_and_stretched_frequencies():
    f, mag = P.frequencies(M.rot(100.0, 8))
    assert mag == 1.0 and all(abs(a - 100.0 ** (-2 * i / 8)) < 1e-15 for i, a in enumerate(f))
    # factor 4 over 64 positions: pairs that turn more than 8 times keep their frequency, those that turn less than half
    # a time have it divided by four, and the factor on cosines and sines is 0.1 ln 4 + 1
    r = M.rot(3000.0, 16, (4.0, 64, 8.0, 0.5))
    f, mag = P.frequencies(r)
    plain = [3000.0 ** (-2 * i / 16) for i in range(8)]
    assert abs(mag - (0.1 * math.log(4.0) + 1)) < 1e-15
    for i, (a, b) in enumerate(zip(f, plain)):
        turns = 64 * b / (2 * math.pi)
        assert b / 4 - 1e-15 <= a <= b + 1e-15
        if turns > 8 * 3000.0 ** (2 / 16):     # a whole index beyond the fast bound
            assert a == b
        if turns < 0.5 / 3000.0 ** (2 / 16):
            assert abs(a - b / 4) < 1e-15
    # a turned pair keeps its length, times the factor; elements behind the turned ones pass
    x = torch.randn(5, 2, 20, dtype=F, generator=torch.Generator().manual_seed(2))
    y = P.rotate_halves(x, r)
    assert torch.equal(y[:, :, 16:], x[:, :, 16:]) and torch.allclose(y[0, :, :16], x[0, :, :16] * mag)
    assert torch.allclose(y[3, 1, 2] ** 2 + y[3, 1, 10] ** 2, (x[3, 1, 2] ** 2 + x[3, 1, 10] ** 2) * mag ** 2)


def test_the_delta_rule_writes_and_reads_a_value():
    """With beta one and no decay a token's value is read back exactly by its own key, and a second write along the same
    key replaces the first."""
    d, dv = 4, 3
    k = torch.tensor([1.0, 0, 0, 0], dtype=F)
    S = torch.zeros(d, dv, dtype=F)
    for v in (torch.tensor([1.0, 2, 3], dtype=F), torch.tensor([-5.0, 0, 7], dtype=F)):
        u = 1.0 * (v - S.T @ k)
        S = S + torch.outer(k, u)
        assert torch.equal(S.T @ k, v)
    # the mixer itself: the state after the first token alone is k u^T, so the first output is u (k . q)
    raw = M.model(11, 8, [M.parallel(M.attn(1, 1, 2, 2, 1.0), M.delta(2, 1, 4, 3, 2), 0.0, 1.0)])
    g = torch.Generator().manual_seed(3)
    names = {"q": (4, 8), "k": (4, 8), "v": (6, 8), "b": (2, 8), "a1": (3, 8), "a2": (8, 3), "g1": (2, 8), "g2": (6, 2), "o": (8, 6),
             "q.conv": (4, 2), "k.conv": (4, 2), "v.conv": (6, 2), "dt_bias": (8,), "A_log": (2,), "norm": (3,)}
    w = {f"p.{n}": torch.randn(*s, generator=g, dtype=F) for n, s in names.items()}
    h = torch.randn(1, 8, generator=g, dtype=F)
    m = raw["layers"][0]["mixer"]["right"]
    out = P.delta_rule_mixer(w, "p", m, h, 1e-5)
    q = P.silu(h @ w["p.q"].T * w["p.q.conv"][:, -1]).reshape(1, 4)
    kk = P.silu(h @ w["p.k"].T * w["p.k.conv"][:, -1]).reshape(1, 4)
    v = P.silu(h @ w["p.v"].T * w["p.v.conv"][:, -1]).reshape(2, 3)
    q = q / torch.sqrt((q * q).sum() + 1e-6) * 0.5
    kk = kk / torch.sqrt((kk * kk).sum() + 1e-6)
    beta = torch.sigmoid(h @ w["p.b"].T).reshape(2, 1)
    o = beta * v * (q * kk).sum()
    gate = torch.sigmoid((h @ w["p.g1"].T) @ w["p.g2"].T).reshape(2, 3)
    want = (P.unit_rms(o, 1e-5) * w["p.norm"] * gate).reshape(1, 6) @ w["p.o"].T
    assert torch.allclose(out, want, atol=1e-12)


def test_the_mixture_takes_the_largest_logits_and_weighs_them_among_themselves():
    g = torch.Generator().manual_seed(4)
    width, E, ff = 6, 5, 4
    f = M.moe(E, 2, ff, shared=3)
    w = {"p.router": torch.randn(E, width, generator=g, dtype=F), "p.router.b": torch.tensor([0.0, 0, 50, 0, 49], dtype=F),
         "p.shared.sg": torch.randn(1, width, generator=g, dtype=F)}
    for e in [f"e{i}" for i in range(E)] + ["shared"]:
        n = 3 if e == "shared" else ff
        w.update({f"p.{e}.gate": torch.randn(n, width, generator=g, dtype=F), f"p.{e}.up": torch.randn(n, width, generator=g, dtype=F),
                  f"p.{e}.down": torch.randn(width, n, generator=g, dtype=F)})
    h = torch.randn(3, width, generator=g, dtype=F) * 0.1
    out = P.mixture(w, "p", f, h)
    z = h @ w["p.router"].T + w["p.router.b"]
    a = torch.softmax(z[:, [2, 4]], dim=1)    # the bias decides the choice, the softmax is over the two alone
    want = a[:, :1] * P.gated_unit(w, "p.e2", h) + a[:, 1:] * P.gated_unit(w, "p.e4", h) + \
        torch.sigmoid(h @ w["p.shared.sg"].T) * P.gated_unit(w, "p.shared", h)
    assert torch.allclose(out, want, atol=1e-12)
    # the gap by which the choice was made: between the second and the third largest logit
    calls = []
    P.mixture(w, "p", f, h, calls)
    third = torch.stack([z[:, e] for e in (0, 1, 3)]).max(0).values
    assert torch.allclose(torch.tensor(calls[0], dtype=F), z[:, [2, 4]].min(1).values - third)


def test_layers_that_read_anothers_keys_use_their_own_queries_and_window(tmp_path):
    from pyre_amd.weights import write_random_model

    write_random_model(tmp_path, config_from_dict(M.SMALL), seed=5, std=0.2, gain_std=0.2)
    cfg, w = P.read_folder(tmp_path)
    ids = list(range(40))
    base = P.forward(w, cfg, ids)
    # the reading layer has no key or value tensors, and a change of the owner's key matrix moves its output
    assert "l2.mix.k" not in w and "l2.mix.q" in w
    other = dict(w)
    other["l0.mix.k"] = w["l0.mix.k"] * 1.5
    assert float((P.forward(other, cfg, ids) - base).abs().max()) > 1e-6
    # its window is its own: tokens further back than the owner's window still reach it
    narrow = copy.deepcopy(cfg)
    narrow["layers"][2]["mixer"]["mask"]["size"] = 20
    assert float((P.forward(w, narrow, ids)[-1] - base[-1]).abs().max()) > 1e-9
