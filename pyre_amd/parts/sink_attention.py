"""Softmax attention over a window with a sink in the denominator, whose projections go through a short causal
convolution over time before they are normed and turned, and whose output is gated element by element."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.attention import STEP_ARRAYS
from pyre_amd.parts.base import (PagedCacheSpec, PagedTensorSpec, SinkAttentionSpec, StateCacheSpec, TensorSpec, make_part,
                                 take)
from pyre_amd.parts.branch import BranchMixer


class SinkAttention(BranchMixer):
    """q, k, v, g = split(h W^T); q, k, v <- conv over time; q, k <- RMS norm per head, turned by position;
    out = softmax over (the window's keys and a sink) of (q k^T scale) v, times sigmoid(g); then the output matrix.

    Keeps two things per request: pages of keys (normed and turned) and values (after the convolution), of which
    those that the window has passed go back to the pool, and the last ``taps - 1`` projected rows, which the
    convolution of the next step's first tokens reads."""

    role = "sattn"

    def __init__(self, spec: SinkAttentionSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("sink attention: heads must be a multiple of kv_heads")
        for name, v in (("key_dim", spec.key_dim), ("value_dim", spec.value_dim)):
            if not (0 < v <= ops.ATTN_MAX_HEAD_DIM):
                raise ValueError(f"sink attention: {name} {v} is outside 1..{ops.ATTN_MAX_HEAD_DIM}")
        if spec.window < 0 or not (0 <= spec.conv_taps <= ops.CONV_MAX_TAPS):
            raise ValueError(f"sink attention: the window must not be negative, the taps lie in 0..{ops.CONV_MAX_TAPS}")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.position = make_part("position", spec.position)
        self.neighbours = getattr(spec.position, "pairing", "halves") == "neighbours"
        self.channels = (spec.num_heads + spec.num_kv_heads) * spec.key_dim + spec.num_kv_heads * spec.value_dim
        self.taps = self.q_gain = self.k_gain = self.sink = None

    def cache_spec(self):
        s = self.spec
        return PagedCacheSpec((PagedTensorSpec("k", (s.num_kv_heads, s.key_dim), token_axis=1),
                               PagedTensorSpec("v", (s.num_kv_heads, s.value_dim), token_axis=1)), s.window)

    def cache_specs(self) -> list:
        specs = [self.cache_spec()]
        if self.spec.conv_taps > 1:
            specs.append(StateCacheSpec((self.spec.conv_taps - 1, self.channels), "float32"))
        return specs

    def step_arrays(self):
        return list(STEP_ARRAYS)

    def in_tensors(self):
        s, p = self.spec, self.spec.prefix
        specs = [TensorSpec(f"{p}.q", (s.num_heads * s.key_dim, s.hidden_size)),
                 TensorSpec(f"{p}.k", (s.num_kv_heads * s.key_dim, s.hidden_size)),
                 TensorSpec(f"{p}.v", (s.num_kv_heads * s.value_dim, s.hidden_size))]
        if s.gated:
            specs.append(TensorSpec(f"{p}.g", (self.inner, s.hidden_size)))
        return specs

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def other_tensors(self):
        s, p = self.spec, self.spec.prefix
        specs = []
        if s.conv_taps:
            # random weights: taps of the order of one, so that every tap matters
            specs += [TensorSpec(f"{p}.{x}.conv", (rows, s.conv_taps), init="normal:0.5")
                      for x, rows in (("q", s.num_heads * s.key_dim), ("k", s.num_kv_heads * s.key_dim),
                                      ("v", s.num_kv_heads * s.value_dim))]
        if s.qk_norm:
            specs += [TensorSpec(f"{p}.q.norm", (s.key_dim,), init="gain"), TensorSpec(f"{p}.k.norm", (s.key_dim,), init="gain")]
        if s.sink:
            specs.append(TensorSpec(f"{p}.sink", (s.num_heads,), init="normal:1.0"))
        return specs

    def bind_others(self, tensors, runtime) -> None:
        s, p = self.spec, self.spec.prefix
        if s.conv_taps:
            # [taps, channels]: a tap's weights of neighbouring channels lie together
            self.taps = torch.cat([take(tensors, f"{p}.{x}.conv").float() for x in ("q", "k", "v")], dim=0).t().contiguous()
        if s.qk_norm:
            self.q_gain = take(tensors, f"{p}.q.norm").float().contiguous()
            self.k_gain = take(tensors, f"{p}.k.norm").float().contiguous()
        if s.sink:
            self.sink = take(tensors, f"{p}.sink").float().contiguous()

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        pages, conv = (cache[0], cache[1]) if isinstance(cache, (list, tuple)) else (cache, None)
        q = ws.get("sattn.q", (n, s.num_heads * s.key_dim), ctx.dtype)
        gate = ws.get("sattn.gate", (n, self.inner), torch.float32) if s.gated else None
        cos, sin, rot = self.position.rotary(ctx.runtime)
        k_pages, v_pages = pages["k"], pages["v"]
        ops.conv_qkv_write(proj, col0, self.taps, conv.tensor if conv is not None else None, ctx.state_slots,
                           ctx.seq_of_token, ctx.q_start, ctx.n_seqs, self.q_gain, self.k_gain, s.norm_eps, cos, sin, rot,
                           self.neighbours, ctx.positions, q, k_pages if pages.writes else None,
                           v_pages if pages.writes else None, gate, pages.slots, n, s.num_heads, s.num_kv_heads, s.key_dim,
                           s.value_dim, pages.page_size)
        shape = (s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, pages.page_size, s.scale, 0.0, None, 0, s.window, 0)
        extra = dict(sink=self.sink, gate_dim=s.value_dim if s.gated else 1)
        tiles = ctx.host.arrays["attention.prefill_tiles"]
        singles = ctx.host.arrays["attention.decode_tokens"]
        if len(tiles) and s.key_dim > ops.ATTN_BIASED_TILE_MAX_KEY_HEAD:
            # key heads that the tile kernel does not hold: every token on its own
            ops.attn_biased_single(q, o, k_pages, v_pages, gate, scale, None, n, ctx.positions, ctx.seq_of_token,
                                   pages.table, *shape, **extra)
            return
        if len(tiles):
            ops.attn_biased_tile(q, o, k_pages, v_pages, gate, scale, ctx.arrays["attention.prefill_tiles"], len(tiles),
                                 ctx.positions, ctx.seq_of_token, pages.table, *shape, **extra)
        if len(singles):
            # a block per span of 128 keys, joined by a second kernel: a step of few tokens fills the chip that way
            spans = ops.attn_biased_spans(pages.table.shape[1], pages.page_size, s.window, 0)
            scratch = None
            if spans > 1:
                scratch = ws.get("sattn.spans", (len(singles) * s.num_heads * spans * (s.value_dim + 2),), torch.float32)
            ops.attn_biased_single(q, o, k_pages, v_pages, gate, scale, ctx.arrays["attention.decode_tokens"],
                                   len(singles), ctx.positions, ctx.seq_of_token, pages.table, *shape, scratch=scratch, **extra)
