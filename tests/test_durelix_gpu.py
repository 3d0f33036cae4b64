"""The Durelix design through the engine against the plain implementation (``plain_durelix``): whole prompts layer by
layer, prefill against token-by-token decoding, portions down to two tokens, mixed batches with pages and slots used
again, long decoding past every window, keys made to stand out at the edges of a window and at page borders, a sink
that decides the output, a state that must survive hundreds of tokens, each mixer alone, the kernels of the norm, the
router and the experts alone, greedy generation through the scheduler, and the programs as processes."""

from __future__ import annotations

import copy
import json
from dataclasses import dataclass
from typing import ClassVar

import numpy as np
import pytest
import torch

import durelix_models as M
import plain_durelix as P
from helpers import cut, first_bad, random_ids, replay
from pyre_amd.config.model import ModelConfig

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

#: bounds on max |difference| / max |logit| of a position, fixed before the first run: float32 against the float64
#: plain run; bfloat16 loosely (the float32 runs are the exact ones)
TOL = {"float32": 2e-5, "bfloat16": 8e-2}
#: a 16-bit run is not compared where the plain router's choice hangs on less than this much of a score
CLOSE_CALL = 0.02
MODELS = {"small": (M.SMALL, 11), "ones": (M.ONES, 12), "wide": (M.WIDE, 13), "odd": (M.ODD, 14),
          # for the 16-bit runs: the routed layer last, so that a close call spoils one position and not the rest
          "small16": (M.routed_last(M.SMALL), 15), "wide16": (M.routed_last(M.WIDE), 16)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from pyre_amd.registry import config_from_dict
    from pyre_amd.weights import write_random_model

    out = {}
    for name, (raw, seed) in MODELS.items():
        d = tmp_path_factory.mktemp("durelix_" + name)
        write_random_model(d, config_from_dict(raw), seed=seed, std=0.2, gain_std=0.2)
        out[name] = (d, *P.read_folder(d))
    return out


def engine_of(folder, dtype, **kw):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=8, max_cached_tokens=1024, max_num_seqs=4, max_num_batched_tokens=512,
                use_graphs=False)
    args.update(kw)
    return Engine.from_folder(folder, EngineConfig(**args))


def plain_rows(cfg, w, ids):
    return P.forward(w, cfg, ids).float()


def whole(reqs):
    return [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()]


def in_portions(reqs, sizes):
    steps = []
    for r, ids in reqs.items():
        pos, parts = 0, cut(len(ids), sizes)
        for k, n in enumerate(parts):
            steps.append(([(r, ids[pos:pos + n], list(range(n)))], [r] if k == len(parts) - 1 else []))
            pos += n
    return steps


def one_by_one(reqs, first):
    steps = []
    for r, ids in reqs.items():
        steps.append(([(r, ids[:first], list(range(first)))], []))
        steps += [([(r, [ids[t]], [0])], [r] if t == len(ids) - 1 else []) for t in range(first, len(ids))]
    return steps


def assert_close(got, want, tol, calls=None):
    """``calls``: request -> :func:`plain_durelix.closest_call` of its tokens (16-bit runs)."""
    if calls is not None:
        # A sequence's first token leaves one term in the recurrent state, and the unit norm of the head's output turns
        # it into sign(q . k) v / rms(v): where q . k happens to be near zero, 16-bit rounding decides the sign, and the
        # row is no measure of the engine. The 32-bit runs compare that position like every other.
        got = {(r, pos): row for (r, pos), row in got.items() if pos != 0 and float(calls[r][pos]) >= CLOSE_CALL}
    bad, worst = first_bad(got, want, tol)
    assert bad is None, bad
    return worst


def calls_of(cfg, w, reqs, dtype):
    return {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()} if dtype == "bfloat16" else None


def all_given_back(eng):
    eng.cache.check_invariants()
    return all(g.allocator.num_used == 0 for g in eng.cache.page_groups) and eng.cache.slots.num_used == 0


# ----------------------------------------------------------------------------- whole prompts, layer by layer


@pytest.mark.parametrize("name", ["small", "ones", "wide", "odd"])
def test_every_layer_of_a_whole_prompt(name, folders):
    from pyre_amd.engine.batch import Entry

    folder, cfg, w = folders[name]
    ids = random_ids(cfg["vocab"], 75, seed=3)
    want, layers = P.forward(w, cfg, ids, return_hidden=True)
    eng = engine_of(folder, "float32")
    seen = {}
    got = eng.step([Entry("a", ids, list(range(len(ids))))], tap=lambda pos, rows: seen.__setitem__(pos, rows.double().cpu()))
    for pos, ref in enumerate(layers):
        d = float((seen[pos] - ref).abs().max() / ref.abs().max())
        assert d <= TOL["float32"], f"layer {pos}: {d:.2e}"
    d = float((got.double().cpu() - want).abs().max() / want.abs().max())
    assert d <= TOL["float32"], d


# (the model of single heads of six and three elements runs in float32 only: in 16 bits its logits are mostly rounding)
@pytest.mark.parametrize("name,dtype,page", [("small", "float32", 8), ("small16", "bfloat16", 16), ("ones", "float32", 4),
                                             ("wide", "float32", 16), ("wide16", "bfloat16", 8), ("odd", "float32", 8),
                                             ("odd", "bfloat16", 16)])
def test_prefill_decode_and_portions_agree_with_plain(name, dtype, page, folders):
    folder, cfg, w = folders[name]
    reqs = {r: random_ids(cfg["vocab"], n, seed=n) for r, n in (("a", 90), ("b", 1), ("c", 37))}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    calls = calls_of(cfg, w, reqs, dtype)
    eng = engine_of(folder, dtype, page_size=page)
    assert_close(replay(eng, whole(reqs)), want, TOL[dtype], calls)
    # most of the prompt, then token by token: the windows pass over decoded tokens
    tail = {r: ids for r, ids in reqs.items() if len(ids) > 1}
    assert_close(replay(eng, one_by_one(tail, 6)), want, TOL[dtype], calls)
    # the first tokens of a sequence one by one from the very start: the convolution's zeros, the table's last row
    assert_close(replay(eng, one_by_one({"c": reqs["c"][:12]}, 1)), want, TOL[dtype], calls)
    for sizes in ([2], [3, 2, 17, 2, 31, 5], [64, 2, 9], [7, 1, 1, 24]):
        assert_close(replay(eng, in_portions(tail, sizes)), want, TOL[dtype], calls)
    assert all_given_back(eng)


@pytest.mark.parametrize("name,dtype,poison", [("small", "float32", True), ("wide", "float32", True), ("small16", "bfloat16", False),
                                               ("ones", "float32", True), ("odd", "float32", True)])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, poison, folders):
    folder, cfg, w = folders[name]
    reqs = {r: random_ids(cfg["vocab"], n, seed=7 * n) for r, n in (("a", 61), ("b", 9), ("c", 100), ("d", 33), ("e", 2), ("f", 47))}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    # three slots, a pool that holds three of the requests at most: everything is used again
    eng = engine_of(folder, dtype, max_num_seqs=3, max_cached_tokens=232, debug_poison=poison)
    fed = {r: 0 for r in reqs}
    live, waiting, steps, k = [], list(reqs), [], 0
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min([5, 1, 13, 2, 1, 40, 1][k % 7], len(reqs[r]) - fed[r])
            k += 1
            entries.append((r, reqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = replay(eng, steps)
    assert_close(got, want, TOL[dtype], calls_of(cfg, w, reqs, dtype))
    assert all_given_back(eng)
    # every request alone gives the same rows, beyond rounding: batch-mates, pages and slots do not matter
    alone = engine_of(folder, dtype)
    for r in ("a", "d"):
        single = replay(alone, whole({r: reqs[r]}))
        for pos in range(len(reqs[r])):
            d = float((single[(r, pos)] - got[(r, pos)]).abs().max() / want[r][pos].abs().max())
            assert d <= (TOL[dtype] if dtype == "float32" else 2 * TOL[dtype]), (r, pos, d)


def test_long_decoding_in_a_pool_that_only_windows_make_fit(folders):
    """260 tokens one by one through a model whose layers all have windows: its pages go back as the windows pass, so a
    pool of 64 tokens is enough; the recurrent branch and the convolution carry on all the while."""
    raw = copy.deepcopy(M.SMALL)
    raw["layers"] = [raw["layers"][0], raw["layers"][2]]
    folder, cfg, w = _folder_of(raw, 21)
    ids = random_ids(cfg["vocab"], 260, seed=1)
    want = {"a": plain_rows(cfg, w, ids)}
    eng = engine_of(folder, "float32", page_size=8, max_cached_tokens=64, max_model_len=512, debug_poison=True)
    assert_close(replay(eng, one_by_one({"a": ids}, 2)), want, TOL["float32"])
    assert eng.cache.page_groups[0].allocator.num_used == 0


_made = {}


def _folder_of(raw, seed, tensors=None):
    """A model folder for ``raw`` (cached by its text); ``tensors(state)`` may change the drawn weights."""
    import tempfile

    from safetensors.torch import save_file

    from pyre_amd.registry import config_from_dict
    from pyre_amd.weights import model_tensor_specs, random_state

    key = (json.dumps(raw, sort_keys=True), seed, tensors)
    if key not in _made:
        d = tempfile.mkdtemp(prefix="durelix_")
        cfg = config_from_dict(raw)
        cfg.save(d)
        state = random_state(model_tensor_specs(cfg), seed, 0.2, 0.2)
        if tensors is not None:
            tensors(state)
        save_file({k: v.contiguous() for k, v in state.items()}, d + "/model.safetensors")
        _made[key] = (d, *P.read_folder(d))
    return _made[key]


# ----------------------------------------------------------------------------- keys made to stand out


#: one layer, a window of 12 tokens on pages of 8, no convolution and no rotation, so that a token's key is the same
#: wherever it stands; a large scale makes the softmax sharp
EDGE = M.model(53, 32, [M.layer(M.left(2, 1, 16, 8, 6.0, window=12), M.right(1, 8, 8, (0.6,)), M.dense(24))], eps=1e-5,
               bigram=(11, 3, 2))


def _keys_like_queries(state):
    # Queries and keys read the first half of a row, values the second; keys are made by the first head's query matrix.
    # Token 51 shares the first half of its row with token 52: its key points where 52's query points, and its value is
    # another. A query of token 52 then gives its weight to itself and to an earlier 51, half each, so that whether the
    # 51 is seen decides its output. The sinks are small beside that.
    q = state["l0.mix.left.q"]
    q[:, 16:] = 0
    state["l0.mix.left.k"] = q[:16].clone()
    state["l0.mix.left.k.norm"] = state["l0.mix.left.q.norm"].clone()
    state["l0.mix.left.v"][:, :16] = 0
    state["l0.mix.left.sink"] = torch.full_like(state["l0.mix.left.sink"], -2.0)
    state["embed"][51, :16] = state["embed"][52, :16]
    state["bigram"] = state["bigram"] * 0.05  # a token's row hardly depends on its neighbour


def test_a_key_just_inside_and_just_outside_the_window():
    folder, cfg, w = _folder_of(EDGE, 31, _keys_like_queries)
    window, T, twin = 12, 52, 51
    eng = engine_of(folder, "float32", page_size=8)
    base = [1 + (i % 50) for i in range(60)]           # no token twice within 50 positions; 51 and 52 appear nowhere
    cases = {"inside": (40, 40 - (window - 1)), "outside": (40, 40 - window), "page_border": (47, 40), "far": (57, 9),
             "next_to_it": (40, 39)}
    reqs = {}
    for name, (i, j) in cases.items():
        ids = list(base)
        ids[i], ids[j] = T, twin
        reqs[name] = ids
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    # the construction works: whether the twin is seen decides the logits at the query
    seen = float((want["inside"][40] - want["outside"][40]).abs().max() / want["inside"][40].abs().max())
    assert seen > 500 * TOL["float32"], seen
    for steps in (whole(reqs), one_by_one(reqs, 30), in_portions(reqs, [39, 2, 5]), in_portions(reqs, [2, 3])):
        assert_close(replay(eng, steps), want, TOL["float32"])
    eng16 = engine_of(folder, "bfloat16", page_size=16)
    for steps in (whole(reqs), one_by_one(reqs, 35)):
        assert_close(replay(eng16, steps), want, TOL["bfloat16"], {r: [1.0] * len(ids) for r, ids in reqs.items()})


def test_a_sink_that_decides_the_output():
    """Sinks as large as the largest scores take half of every query's weight: leaving them out, scaling them or
    counting them twice would move the logits far beyond rounding."""
    def big_sinks(state):
        state["l0.mix.left.sink"] = torch.tensor([4.0, 1.0], dtype=state["l0.mix.left.sink"].dtype)
    folder, cfg, w = _folder_of(EDGE, 33, big_sinks)
    reqs = {"a": random_ids(cfg["vocab"], 50, seed=4), "b": random_ids(cfg["vocab"], 3, seed=5)}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    without = dict(w)
    without["l0.mix.left.sink"] = torch.full_like(w["l0.mix.left.sink"], -80.0)
    moved = float((plain_rows(cfg, without, reqs["a"]) - want["a"]).abs().max() / want["a"].abs().max())
    assert moved > 500 * TOL["float32"], moved
    eng = engine_of(folder, "float32", page_size=8)
    for steps in (whole(reqs), one_by_one(reqs, 2), in_portions(reqs, [2, 7])):
        assert_close(replay(eng, steps), want, TOL["float32"])


def test_a_state_that_has_to_last():
    """Decays close to one and exactly one: the first tokens reach the last logits through the recurrent state alone
    (the window is 12 tokens, the changed token is the fourth)."""
    raw = copy.deepcopy(EDGE)
    raw["layers"][0]["mixer"]["right"] = M.right(2, 8, 8, (0.9995, 1.0), rot=(10000.0, 4))
    raw["layers"][0]["mixer"]["left"]["conv"] = 3
    folder, cfg, w = _folder_of(raw, 32)
    ids = random_ids(cfg["vocab"], 300, seed=9)
    other = list(ids)
    other[3] = (ids[3] + 1) % cfg["vocab"]
    want = {"a": plain_rows(cfg, w, ids), "b": plain_rows(cfg, w, other)}
    moved = float((want["a"][-1] - want["b"][-1]).abs().max() / want["a"][-1].abs().max())
    assert moved > 1e-3, moved
    eng = engine_of(folder, "float32", page_size=16, max_cached_tokens=640)
    reqs = {"a": ids, "b": other}
    assert_close(replay(eng, whole(reqs)), want, TOL["float32"])
    assert_close(replay(eng, in_portions(reqs, [64, 2, 31, 100, 3])), want, TOL["float32"])
    assert_close(replay(eng, one_by_one({"a": ids}, 30)), want, TOL["float32"])


# ----------------------------------------------------------------------------- each mechanism alone


@dataclass(frozen=True)
class OneBranchConfig(ModelConfig):
    """A model of post-norm layers whose mixer is a single branch: 'left' or 'right' of the design."""

    raw: dict
    architecture: ClassVar[str] = "ToyOneBranch"

    @classmethod
    def from_dict(cls, raw):
        return cls(raw)

    def to_dict(self):
        return self.raw

    def save(self, folder):
        import pathlib
        pathlib.Path(folder, "config.json").write_text(json.dumps(self.raw))

    def __hash__(self):
        return id(self)


def _build_one_branch(cfg):
    from pyre_amd.config.durelix import RetentionConfig, SinkAttentionConfig
    from pyre_amd.parts.base import (EmbeddingSpec, LayerCall, LMHeadSpec, ModelSpec, NoPositionSpec, PostNormBlockSpec,
                                     RetentionSpec, RMSNormSpec, RotarySpec, SinkAttentionSpec)

    raw = cfg.raw
    width, eps = raw["width"], raw["norm"]["eps"]

    def position(dim, base, dims, pairing):
        return RotarySpec(dim, base, 0, rotary_dim=dims, exact=True, pairing=pairing) if dims else NoPositionSpec()

    layers = []
    for i, layer in enumerate(raw["layers"]):
        p = f"l{i}.mix"
        if layer["type"] == "left":
            a = SinkAttentionConfig.from_dict(layer["mixer"], "left")
            mixer = SinkAttentionSpec(width, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, position(a.dim, a.rot_base, a.rot_dims, "neighbours"),
                                      p, window=a.window, conv_taps=a.conv, norm_eps=eps)
        else:
            r = RetentionConfig.from_dict(layer["mixer"], "right")
            mixer = RetentionSpec(width, r.heads, r.dim, r.vdim, r.decay, position(r.dim, r.rot_base, r.rot_dims, "halves"), p, norm_eps=eps)
        layers.append(PostNormBlockSpec(mixer, RMSNormSpec(width, eps, "", name=f"l{i}.norm1")))
    return ModelSpec(width, raw["vocab"], 0, EmbeddingSpec(raw["vocab"], width, name="embed"), tuple(layers),
                     tuple(LayerCall(i) for i in range(len(layers))), RMSNormSpec(width, eps, "", name="final.norm"),
                     LMHeadSpec(raw["vocab"], width, name="embed"))


@pytest.mark.parametrize("kind", ["left", "right"])
def test_each_mixer_alone(kind, tmp_path):
    from pyre_amd.registry import register_architecture, unregister_architecture
    from pyre_amd.weights import write_random_model

    # (nine taps: more than the kernel with four elements a lane takes, and more than the first portions are long)
    mixers = {"left": [M.left(4, 2, 24, 16, 0.5, window=20, conv=3, rot=(100.0, 10)), M.left(5, 1, 7, 9, 0.8),
                       M.left(2, 1, 12, 8, 0.6, window=5, conv=9, rot=(10.0, 4))],
              "right": [M.right(2, 16, 24, (0.9, 0.99), rot=(30.0, 16)), M.right(3, 33, 7, (1.0, 0.3, 0.97))]}[kind]
    raw = {"architectures": ["ToyOneBranch"], "vocab": 71, "width": 40, "norm": {"eps": 1e-5},
           "layers": [{"type": kind, "mixer": m, "mlp": None} for m in mixers]}
    P.MIXERS["left"] = P.sink_attention
    P.MIXERS["right"] = P.retention
    register_architecture(OneBranchConfig.architecture, OneBranchConfig, _build_one_branch)
    try:
        write_random_model(tmp_path, OneBranchConfig(raw), seed=41, std=0.2, gain_std=0.2)
        cfg, w = P.read_folder(tmp_path)
        reqs = {r: random_ids(71, n, seed=n) for r, n in (("a", 70), ("b", 19))}
        want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
        eng = engine_of(tmp_path, "float32")
        kinds = [[type(s).__name__ for s in c] for c in eng.model.cache_specs()]
        assert kinds == ([["PagedCacheSpec", "StateCacheSpec"], ["PagedCacheSpec"], ["PagedCacheSpec", "StateCacheSpec"]]
                         if kind == "left" else [["StateCacheSpec"]] * 2)
        assert_close(replay(eng, whole(reqs)), want, TOL["float32"])
        assert_close(replay(eng, in_portions(reqs, [5, 2, 30])), want, TOL["float32"])
        assert_close(replay(eng, one_by_one(reqs, 4)), want, TOL["float32"])
    finally:
        unregister_architecture(OneBranchConfig.architecture)
        P.MIXERS.pop("left"), P.MIXERS.pop("right")


@pytest.mark.parametrize("hidden,dtype", [(50, torch.float32), (48, torch.float32), (700, torch.float32), (2100, torch.bfloat16),
                                          (5000, torch.float32)])
def test_the_residual_sum_with_normed_terms(hidden, dtype):
    """Two terms, each with a norm and a factor of its own, their sum normed again, added to the stream, the stream
    handed on as it is or normed once more; with fewer of these; for listed rows only."""
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(hidden)
    n = 9
    resid = torch.randn(n, hidden, generator=g) * 3 + 1.5
    a, b = torch.randn(3, n, hidden, generator=g), torch.randn(1, n, hidden, generator=g) * 4
    ga, gb, go, gn = ((1 + 0.3 * torch.randn(hidden, generator=g)).to(dtype) for _ in range(4))
    dd = lambda t: t.double()  # noqa: E731
    term = 0.5 * P.rms_norm(dd(a).sum(0), dd(ga), 1e-4) + 0.25 * P.rms_norm(dd(b).sum(0), dd(gb), 1e-4)
    want_resid = dd(resid) + P.rms_norm(term, dd(go), 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 1e-2

    def pending(outer=True):
        second = ops.Partials(b.to(DEV), None, ops.PostNorm(gb.to(DEV), 1e-4, kind="rms"), 0.25)
        return ops.Partials(a.to(DEV), None, ops.PostNorm(ga.to(DEV), 1e-4, kind="rms"), 0.5, second,
                            ops.PostNorm(go.to(DEV), 1e-5, kind="rms") if outer else None)

    r = resid.to(DEV)
    out = torch.empty(n, hidden, device=DEV, dtype=dtype)
    ops.add_rms_terms(r, pending(), None, 0.0, out)
    assert float((r.cpu().double() - want_resid).abs().max()) < 1e-5 * float(want_resid.abs().max())
    assert float((out.cpu().double() - want_resid).abs().max()) < tol * float(want_resid.abs().max())
    # the stream normed as it is handed on; the listed rows only, the stream untouched
    r2 = resid.to(DEV)
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    out2 = torch.empty(3, hidden, device=DEV, dtype=dtype)
    ops.add_rms_terms(r2, pending(), gn.to(DEV), 1e-6, out2, rows)
    want2 = P.rms_norm(want_resid, dd(gn), 1e-6)[[7, 0, 3]]
    assert torch.equal(r2.cpu(), resid) and float((out2.cpu().double() - want2).abs().max()) < tol * float(want2.abs().max())
    # one plain term under a norm of the sum (a feed-forward's result); no term at all
    r3 = resid.to(DEV)
    ops.add_rms_terms(r3, ops.Partials(a.to(DEV), outer=ops.PostNorm(go.to(DEV), 1e-5, kind="rms")), None, 0.0, out)
    want3 = dd(resid) + P.rms_norm(dd(a).sum(0), dd(go), 1e-5)
    assert float((r3.cpu().double() - want3).abs().max()) < 1e-5 * float(want3.abs().max())
    r4 = resid.to(DEV)
    ops.add_rms_terms(r4, None, None, 0.0, out)
    assert torch.equal(r4.cpu(), resid) and float((out.cpu().double() - dd(resid)).abs().max()) < tol * float(resid.abs().max())
    # the same through the norm part, which also takes the plain case
    with pytest.raises(Exception):
        ops.add_rmsnorm(r, pending(), gn.to(DEV), 1e-6, out)
    with pytest.raises(Exception):
        ops.add_layernorm(r, pending(), gn.to(DEV), 1e-6, out)


@pytest.mark.parametrize("experts,top,groups,keep", [(6, 2, 3, 1), (10, 3, 2, 1), (8, 8, 1, 1), (12, 4, 4, 2), (130, 5, 10, 3), (3, 1, 3, 3)])
def test_the_routing_kernel(experts, top, groups, keep):
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(experts)
    n = 40
    z = torch.randn(2, n, experts, generator=g) * 2
    z[:, 5] = z[:, 5].round()            # rows with equal logits: the lower index wins
    z[:, 6] = 0.0
    corr = torch.randn(experts, generator=g) * 0.3 - 0.5   # mostly negative choice scores
    gates = torch.full((n, experts), -1.0, device=DEV)
    ops.route_grouped(ops.Partials(z.to(DEV)), corr.to(DEV), gates, n, top, groups, keep)
    gates = gates.cpu().double()
    close = 0
    for t in range(n):
        s = torch.softmax(z[:, t].double().sum(0), -1)
        chosen, gap = P.choose(s, corr.double(), top, groups, keep)
        if 0 < gap < 1e-6:
            close += 1
            continue
        want = torch.zeros(experts, dtype=torch.float64)
        want[chosen] = s[chosen]
        assert float((gates[t] - want).abs().max()) < 1e-6, (t, chosen, gates[t].nonzero().flatten().tolist())
    assert close < 3


def test_the_experts_activation_and_the_identity_experts():
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(8)
    n, experts, ff, width = 7, 3, 10, 26
    gu = torch.randn(2, n, 2 * experts * ff, generator=g)
    gates = torch.rand(n, experts + 2, generator=g)
    gates[gates < 0.4] = 0.0
    total = gu.double().sum(0)
    gate, up = total[:, :experts * ff], total[:, experts * ff:]
    want = gates.double()[:, :experts].repeat_interleave(ff, 1) * P.silu(gate) * up
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        out = torch.empty(n, experts * ff, device=DEV, dtype=dtype)
        ops.expert_glu_act(ops.Partials(gu.to(DEV)), gates.to(DEV), out, n, experts, ff)
        assert float((out.cpu().double() - want).abs().max()) < tol * float(want.abs().max())
        p = torch.randn(2, n, width, generator=g)
        h = torch.randn(n, width, generator=g).to(dtype)
        pd = p.to(DEV)
        ops.add_weighted_rows(ops.Partials(pd), h.to(DEV), gates.to(DEV), experts, 2, n)
        want_p = p.double().sum(0) + gates.double()[:, experts:].sum(1, keepdim=True) * h.double()
        assert float((pd.sum(0).cpu().double() - want_p).abs().max()) < 1e-5
    up1 = torch.randn(3, n, 37, generator=g)
    act = torch.empty(n, 37, device=DEV)
    ops.relu2(ops.Partials(up1.to(DEV)), act, n)
    assert float((act.cpu().double() - torch.relu(up1.double().sum(0)) ** 2).abs().max()) < 1e-5


# ----------------------------------------------------------------------------- the entry points


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(graphs, folders):
    """The scheduler runs one step ahead, its tokens fed on the device: the previous token of the second embedding
    table is state on the device too. With graphs the decode steps are captured and replayed."""
    from pyre_amd.api import generate, load_model

    folder, cfg, w = folders["small"]
    prompts = [random_ids(cfg["vocab"], n, seed=n + 1) for n in (1, 9, 40, 23)]
    eng, _ = load_model(str(folder), device=DEV, dtype="float32", page_size=8, max_cached_tokens=1024, max_num_seqs=4,
                        max_num_batched_tokens=64, prefill_chunk=16, use_graphs=graphs)
    got = generate(eng, prompts, max_new_tokens=30)
    for p, g in zip(prompts, got):
        assert len(g) == 30
        ids = list(p)
        for k, tok in enumerate(g):
            row = P.forward(w, cfg, ids)[-1]
            twin = int(row.argmax())
            if twin != tok:
                margin = float((row[twin] - row[tok]) / row.abs().max())
                assert margin < TOL["float32"], f"token {k} is {tok}, plainly {twin} (margin {margin:.2e})"
            ids.append(tok)
    assert all_given_back(eng)
    if graphs:
        assert eng.graph_replays > 0


def test_the_generate_program_as_a_process(folders, tmp_path):
    import subprocess
    import sys
    from pathlib import Path

    folder, cfg, w = folders["odd"]
    root = Path(__file__).resolve().parent.parent
    out = tmp_path / "res.json"
    proc = subprocess.run([sys.executable, str(root / "bin" / "pyre_generate"), "--model", str(folder), "--dtype", "float32",
                           "--prompt-ids", "7,3,3,41,9,50,5", "--prompt-ids", "11", "--tokens", "12", "--num-blocks", "32",
                           "--max-batch", "2", "--out", str(out)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    res = json.loads(out.read_text())
    assert res["dtype"] == "float32" and [len(g) for g in res["generated"]] == [12, 12]
    for prompt, tokens in zip(res["prompts"], res["generated"]):
        ids = list(prompt)
        for k, tok in enumerate(tokens):
            row = P.forward(w, cfg, ids)[-1]
            twin = int(row.argmax())
            if twin != tok:
                margin = float((row[twin] - row[tok]) / row.abs().max())
                assert margin < TOL["float32"], f"token {k} is {tok}, plainly {twin} (margin {margin:.2e})"
            ids.append(tok)


@pytest.mark.parametrize("dtype,extra", [("float32", ("--page-size", "8", "--poison")), ("bfloat16", ("--graphs",))])
def test_trace_run_as_a_process(dtype, extra, folders, tmp_path):
    from test_trace_run_gpu import run_trace

    folder, cfg, w = folders["small" if dtype == "float32" else "small16"]
    vocab = cfg["vocab"]
    reqs = {"a": random_ids(vocab, 70, 1), "b": random_ids(vocab, 40, 2), "c": random_ids(vocab, 64, 3), "d": random_ids(vocab, 3, 4),
            "e": random_ids(vocab, 61, 5)}
    fed = {r: 0 for r in reqs}
    sizes = [13, 2, 30, 1, 7, 64, 3]
    live, waiting, steps, k, wanted = [], list(reqs), [], 0, {}
    while live or waiting:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min(sizes[k % len(sizes)], len(reqs[r]) - fed[r])
            k += 1
            want = [] if k % 5 == 0 else list(range(0, n, 2))
            entries.append({"id": r, "tokens": reqs[r][fed[r]:fed[r] + n], "want": want})
            wanted.setdefault(len(steps), []).extend((r, fed[r] + x) for x in want)
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    out = tmp_path / "out"
    run_trace(folder, dtype, out, 4 * 128, steps, extra)
    ref = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    calls = {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()}
    checked = 0
    for st, rows in wanted.items():
        if not rows:
            assert not (out / f"{st}.f32").exists()
            continue
        got = torch.from_numpy(np.fromfile(out / f"{st}.f32", dtype="<f4").reshape(len(rows), vocab))
        for i, (r, pos) in enumerate(rows):
            if dtype == "bfloat16" and (pos == 0 or float(calls[r][pos]) < CLOSE_CALL):
                continue  # see assert_close
            d = float((got[i] - ref[r][pos]).abs().max() / ref[r][pos].abs().max())
            assert d <= TOL[dtype], f"step {st} request {r} position {pos}: {d:.3e}"
            checked += 1
    assert checked > 50
