"""Grouped softmax attention over a window with biased projections, whose queries and keys may be normed over their whole
projection, whose softmax may hold a sink of score zero, and which may read another layer's keys and values."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.attention import STEP_ARRAYS
from pyre_amd.parts.base import PagedCacheSpec, PagedTensorSpec, TensorSpec, WindowAttentionSpec, make_part, take
from pyre_amd.parts.branch import BranchMixer


class WindowAttention(BranchMixer):
    """q, k, v = split(h W^T + b); q, k <- RMS norm over the whole projection (if the description says so), turned by
    position; out = softmax over the window's keys (and a sink of score zero, if it says so) of (q k^T scale) v; then the
    output matrix.

    Keeps pages of keys (normed and turned) and values, of which those that the window has passed go back to the pool.
    A layer without key and value projections of its own runs its queries against the pages of the layer that the order of
    layers names, with its own window."""

    role = "wattn"

    def __init__(self, spec: WindowAttentionSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("window attention: heads must be a multiple of kv_heads")
        for name, v in (("key_dim", spec.key_dim), ("value_dim", spec.value_dim)):
            if not (0 < v <= ops.ATTN_MAX_HEAD_DIM):
                raise ValueError(f"window attention: {name} {v} is outside 1..{ops.ATTN_MAX_HEAD_DIM}")
        if spec.window < 0 or (spec.cache_window is not None and spec.cache_window < 0):
            raise ValueError("window attention: a window must not be negative")
        if spec.sink not in ("none", "zero"):
            raise ValueError(f"window attention: sink is 'none' or 'zero', not {spec.sink!r}")
        if getattr(spec.position, "pairing", "halves") != "halves":
            raise ValueError("window attention: its kernel turns element e with e + rot/2")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.position = make_part("position", spec.position)
        self.q_gain = self.k_gain = self.sink = None

    def cache_spec(self):
        s = self.spec
        window = s.window if s.cache_window is None else s.cache_window
        return PagedCacheSpec((PagedTensorSpec("k", (s.num_kv_heads, s.key_dim), token_axis=1),
                               PagedTensorSpec("v", (s.num_kv_heads, s.value_dim), token_axis=1)), window)

    def step_arrays(self):
        return list(STEP_ARRAYS)

    def _projections(self):
        s = self.spec
        rows = [("q", s.num_heads * s.key_dim)]
        if s.own_kv:
            rows += [("k", s.num_kv_heads * s.key_dim), ("v", s.num_kv_heads * s.value_dim)]
        return rows

    def in_tensors(self):
        s = self.spec
        return [TensorSpec(f"{s.prefix}.{x}", (rows, s.hidden_size)) for x, rows in self._projections()]

    def in_biases(self):
        s = self.spec
        return [TensorSpec(f"{s.prefix}.{x}.b", (rows,)) if s.qkv_bias else None for x, rows in self._projections()]

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def out_bias(self):
        return TensorSpec(f"{self.spec.prefix}.o.b", (self.spec.hidden_size,)) if self.spec.out_bias else None

    def other_tensors(self):
        s = self.spec
        if not s.wide_norm:
            return []
        return [TensorSpec(f"{s.prefix}.{x}.norm", (rows,), init="gain") for x, rows in self._projections() if x != "v"]

    def bind_others(self, tensors, runtime) -> None:
        s = self.spec
        if s.wide_norm:
            self.q_gain = take(tensors, f"{s.prefix}.q.norm").float().contiguous()
            if s.own_kv:
                self.k_gain = take(tensors, f"{s.prefix}.k.norm").float().contiguous()
        if s.sink == "zero":
            self.sink = torch.zeros(s.num_heads, dtype=torch.float32, device=runtime.device)

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        pages = cache[0] if isinstance(cache, (list, tuple)) else cache
        q = ws.get("wattn.q", (n, s.num_heads * s.key_dim), ctx.dtype)
        cos, sin, rot = self.position.rotary(ctx.runtime)
        k_pages, v_pages = pages["k"], pages["v"]
        if pages.writes != s.own_kv:
            raise ValueError("window attention: a layer writes the pages it has projections for, and no others")
        ops.wide_norm_qkv_write(proj, col0, self.q_gain, self.k_gain, s.norm_eps, cos, sin, rot, ctx.positions, q,
                                k_pages if s.own_kv else None, v_pages if s.own_kv else None, pages.slots, n, s.num_heads,
                                s.num_kv_heads if s.own_kv else 0, s.key_dim, s.value_dim, pages.page_size)
        shape = (s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim, pages.page_size, s.scale, 0.0, None, 0, s.window, 0)
        extra = dict(sink=self.sink, gate_dim=1)
        tiles = ctx.host.arrays["attention.prefill_tiles"]
        singles = ctx.host.arrays["attention.decode_tokens"]
        if len(tiles) and s.key_dim > ops.ATTN_BIASED_TILE_MAX_KEY_HEAD:
            # key heads that the tile kernel does not hold: every token on its own
            ops.attn_biased_single(q, o, k_pages, v_pages, None, scale, None, n, ctx.positions, ctx.seq_of_token,
                                   pages.table, *shape, **extra)
            return
        if len(tiles):
            ops.attn_biased_tile(q, o, k_pages, v_pages, None, scale, ctx.arrays["attention.prefill_tiles"], len(tiles),
                                 ctx.positions, ctx.seq_of_token, pages.table, *shape, **extra)
        if len(singles):
            # a block per span of 128 keys, joined by a second kernel: a step of few tokens fills the chip that way
            spans = ops.attn_biased_spans(pages.table.shape[1], pages.page_size, s.window, 0)
            scratch = None
            if spans > 1:
                scratch = ws.get("wattn.spans", (len(singles) * s.num_heads * spans * (s.value_dim + 2),), torch.float32)
            ops.attn_biased_single(q, o, k_pages, v_pages, None, scale, ctx.arrays["attention.decode_tokens"],
                                   len(singles), ctx.positions, ctx.seq_of_token, pages.table, *shape, scratch=scratch, **extra)
