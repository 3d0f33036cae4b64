"""The Zorulix design as a list of parts.

Pre-norm layers with an RMS norm whose weight is stored around zero, x += mixer(norm1(x)), x += ff(norm2(x)), and behind
them a third sublayer fed by the token itself: a slice of a second token table, gated by a narrow product of the stream,
carried to the width and RMS-normed with a plain weight. The embedding's rows are scaled. A layer's mixer is one of two.
'attention': grouped softmax attention over a window with biased projections, queries and keys RMS-normed over their whole
projection before they are turned by position (part of a head, element e with e + dims/2), a sink of score zero in the
softmax's denominator; a layer with ``kv_from`` has no key and value projections and reads the pages of the layer it
names. 'parallel': two mixers side by side on the same rows, their scaled results summed: the same attention without norm
and sink, with an output bias and frequencies that may be stretched for long contexts, and the gated delta rule (a
float32 matrix state per head behind a short convolution). The feed-forward is a mixture of gated experts whose chosen
logits are weighted by their own softmax, with a shared expert behind a sigmoid gate per token; or absent. Tensor names:
``embed``, ``side.embed``, ``final.norm``, ``head``, ``l<i>.norm1 / norm2``, ``l<i>.mix.*`` (``.left.*``, ``.right.*``),
``l<i>.mlp.*``, ``l<i>.side.*``.
"""

from __future__ import annotations

from pyre_amd.config.zorulix import AttentionConfig, MixtureConfig, ParallelConfig, ZorulixConfig
from pyre_amd.parts.base import (BlockSpec, EmbeddingSpec, GatedDeltaRuleSpec, LayerCall, LMHeadSpec, ModelSpec,
                                 NoPositionSpec, ParallelMixerSpec, RMSNormSpec, RotarySpec, SoftmaxTopKMoESpec,
                                 TokenSideSpec, WindowAttentionSpec)
from pyre_amd.registry import register_architecture

#: beside the sum of squares where the recurrent branch makes its queries and keys unit vectors
UNIT_EPS = 1e-6


def _position(m: AttentionConfig):
    r = m.rot
    if r is None:
        return NoPositionSpec()
    return RotarySpec(m.dim, r.base, 0, rotary_dim=r.dims, exact=True, scaling=r.scaling)


def _cache_window(cfg: ZorulixConfig, i: int, m: AttentionConfig) -> int | None:
    """The window by which layer i's pages are given back: its own, or the widest of the layers that read them."""
    windows = [m.window] + [l.mixer.window for l in cfg.layers if getattr(l.mixer, "kv_from", None) == i]
    keep = 0 if 0 in windows else max(windows)
    return None if keep == m.window else keep


def _attention(cfg: ZorulixConfig, i: int, m: AttentionConfig, prefix: str) -> WindowAttentionSpec:
    return WindowAttentionSpec(cfg.width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, _position(m), prefix,
                               window=m.window, qkv_bias=True, out_bias=False, wide_norm=True, norm_eps=cfg.norm_eps,
                               sink="zero", own_kv=m.kv_from is None, cache_window=_cache_window(cfg, i, m))


def _parallel(cfg: ZorulixConfig, i: int, m: ParallelConfig, prefix: str) -> ParallelMixerSpec:
    a, r = m.left, m.right
    left = WindowAttentionSpec(cfg.width, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, _position(a), f"{prefix}.left",
                               window=a.window, qkv_bias=True, out_bias=True, wide_norm=False, norm_eps=cfg.norm_eps,
                               sink="none")
    right = GatedDeltaRuleSpec(cfg.width, r.heads, r.kv_heads, r.dim, r.vdim, r.conv, f"{prefix}.right",
                               norm_eps=cfg.norm_eps, unit_eps=UNIT_EPS)
    return ParallelMixerSpec(cfg.width, (left, right), (m.left_scale, m.right_scale))


MIXERS = {AttentionConfig: _attention, ParallelConfig: _parallel}


def _mixture(cfg: ZorulixConfig, f: MixtureConfig, prefix: str) -> SoftmaxTopKMoESpec:
    return SoftmaxTopKMoESpec(cfg.width, f.experts, f.top, f.expert_ff, prefix, shared_size=f.shared_ff, shared_gate=True,
                              router_bias=True)


FEED_FORWARDS = {MixtureConfig: _mixture}


def build_zorulix(cfg: ZorulixConfig) -> ModelSpec:
    def norm(name):
        return RMSNormSpec(cfg.width, cfg.norm_eps, "", name=name, one_plus=True)

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = {}
        if layer.mlp is not None:
            ff = dict(feed_forward=FEED_FORWARDS[type(layer.mlp)](cfg, layer.mlp, f"{p}.mlp"), feed_forward_norm=norm(f"{p}.norm2"))
        side = {}
        if cfg.side_dim:
            side = dict(token_input=TokenSideSpec(cfg.width, cfg.vocab, cfg.side_dim, "side.embed",
                                                  cfg.side_dim * len(cfg.layers), i * cfg.side_dim, f"{p}.side"),
                        token_input_norm=RMSNormSpec(cfg.width, cfg.norm_eps, "", name=f"{p}.side.norm"))
        layers.append(BlockSpec(mixer=MIXERS[type(layer.mixer)](cfg, i, layer.mixer, f"{p}.mix"), mixer_norm=norm(f"{p}.norm1"),
                                feed_forward=ff.get("feed_forward"), feed_forward_norm=ff.get("feed_forward_norm"), **side))
        schedule.append(LayerCall(i, cache_from=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=0,
                     embedding=EmbeddingSpec(cfg.vocab, cfg.width, name="embed", scale=cfg.embedding_scale),
                     layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"),
                     head=LMHeadSpec(cfg.vocab, cfg.width, name="head"))


register_architecture(ZorulixConfig.architecture, ZorulixConfig, build_zorulix)
