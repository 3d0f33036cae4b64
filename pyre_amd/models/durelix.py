"""The Durelix design as a list of parts.

Every sublayer reads the residual stream itself and only its result is normed (RMS norm with a gain) before it joins
the stream. The mixer of a 'parallel' layer is two mixers side by side on the same rows, each with an output matrix of
its own, each result normed over the width with a gain of its own, half their sum handed on: softmax attention over a
window with a sink in the denominator (projections through a short causal convolution, queries and keys normed per
head and turned in neighbouring pairs, a sigmoid gate per output element) and retention (linear attention with a fixed
decay per head, queries and keys turned in halves, a float32 matrix state per head). The feed-forward is
down(relu(up x)^2), or a mixture of gated units whose router scores are a softmax, corrected for the choice, limited
to the best groups, with experts that hand their input back; or absent. The token embedding is joined by a row of a
second table chosen by the pair (previous token, token); the head is the embedding table. Tensor names: ``embed``,
``bigram``, ``final.norm``, ``l<i>.norm1 / norm2``, ``l<i>.mix.left.*``, ``l<i>.mix.right.*``, ``l<i>.mix.left.out /
right.out``, ``l<i>.mlp.*``.
"""

from __future__ import annotations

from pyre_amd.config.durelix import DenseConfig, DurelixConfig, MixtureConfig, ParallelMixerConfig
from pyre_amd.parts.base import (BigramEmbeddingSpec, EmbeddingSpec, GroupedSoftmaxMoESpec, LayerCall, LMHeadSpec, ModelSpec,
                                 NoPositionSpec, ParallelMixerSpec, PostNormBlockSpec, ReluSquaredMLPSpec, RetentionSpec,
                                 RMSNormSpec, RotarySpec, SinkAttentionSpec)
from pyre_amd.registry import register_architecture

#: the two branches' normed results are averaged
BRANCH_SCALE = 0.5


def _position(dim: int, base: float, dims: int, pairing: str):
    return RotarySpec(dim, base, 0, rotary_dim=dims, exact=True, pairing=pairing) if dims else NoPositionSpec()


def _parallel(cfg: DurelixConfig, m: ParallelMixerConfig, prefix: str) -> ParallelMixerSpec:
    a, r = m.left, m.right
    left = SinkAttentionSpec(cfg.width, a.heads, a.kv_heads, a.dim, a.vdim, a.scale,
                             _position(a.dim, a.rot_base, a.rot_dims, "neighbours"), f"{prefix}.left", window=a.window,
                             conv_taps=a.conv, qk_norm=True, norm_eps=cfg.norm_eps, sink=True, gated=True)
    right = RetentionSpec(cfg.width, r.heads, r.dim, r.vdim, r.decay, _position(r.dim, r.rot_base, r.rot_dims, "halves"),
                          f"{prefix}.right", norm_eps=cfg.norm_eps)
    return ParallelMixerSpec(cfg.width, (left, right), (BRANCH_SCALE, BRANCH_SCALE),
                             out_norms=(f"{prefix}.left.out", f"{prefix}.right.out"), norm_eps=cfg.norm_eps)


MIXERS = {ParallelMixerConfig: _parallel}


def _dense(cfg: DurelixConfig, f: DenseConfig, prefix: str) -> ReluSquaredMLPSpec:
    return ReluSquaredMLPSpec(cfg.width, f.ff, prefix)


def _mixture(cfg: DurelixConfig, f: MixtureConfig, prefix: str) -> GroupedSoftmaxMoESpec:
    return GroupedSoftmaxMoESpec(cfg.width, f.experts, f.top, f.expert_ff, prefix, identity=f.identity, groups=f.groups,
                                 keep_groups=f.keep_groups)


FEED_FORWARDS = {DenseConfig: _dense, MixtureConfig: _mixture}


def build_durelix(cfg: DurelixConfig) -> ModelSpec:
    def norm(name):
        return RMSNormSpec(cfg.width, cfg.norm_eps, "", name=name)

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = {}
        if layer.mlp is not None:
            ff = dict(feed_forward=FEED_FORWARDS[type(layer.mlp)](cfg, layer.mlp, f"{p}.mlp"),
                      feed_forward_post_norm=norm(f"{p}.norm2"))
        layers.append(PostNormBlockSpec(mixer=MIXERS[type(layer.mixer)](cfg, layer.mixer, f"{p}.mix"),
                                        mixer_post_norm=norm(f"{p}.norm1"), **ff))
    b = cfg.bigram
    embedding = EmbeddingSpec(cfg.vocab, cfg.width, name="embed") if b is None else \
        BigramEmbeddingSpec(cfg.vocab, cfg.width, b.buckets, b.mul_prev, b.mul_cur, name="embed", pairs_name="bigram")
    return ModelSpec(hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=0, embedding=embedding,
                     layers=tuple(layers), schedule=tuple(LayerCall(i) for i in range(len(layers))),
                     final_norm=norm("final.norm"), head=LMHeadSpec(cfg.vocab, cfg.width, name=embedding.name))


register_architecture(DurelixConfig.architecture, DurelixConfig, build_durelix)
