"""Gated linear attention: a float32 matrix state per head and request, decayed per key channel."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
import math

from pyre_amd.parts.base import GatedLinearAttentionSpec, RetentionSpec, StateCacheSpec, TensorSpec, make_part, take
from pyre_amd.parts.branch import BranchMixer

#: columns of the decay's low-rank product that the random-weights mode draws when a description leaves them to the file
DEFAULT_RANK = 8


class GatedLinearAttention(BranchMixer):
    role = "gla"

    def __init__(self, spec: GatedLinearAttentionSpec):
        if not (0 < spec.key_dim <= ops.GLA_MAX_KEY_HEAD and 0 < spec.value_dim <= ops.GLA_MAX_VALUE_HEAD):
            raise ValueError(f"gated linear attention: head sizes {spec.key_dim} / {spec.value_dim} are outside "
                             f"1..{ops.GLA_MAX_KEY_HEAD} / 1..{ops.GLA_MAX_VALUE_HEAD}")
        if not (spec.tau > 0) or spec.num_heads <= 0:
            raise ValueError("gated linear attention: tau and heads must be positive")
        if spec.rank is not None and not (0 < spec.rank <= ops.GLA_MAX_RANK):
            raise ValueError(f"gated linear attention: rank {spec.rank} is outside 1..{ops.GLA_MAX_RANK}")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.a2 = self.a2_bias = self.gain = None

    def cache_spec(self):
        s = self.spec
        return StateCacheSpec((s.num_heads, s.key_dim, s.value_dim), "float32")

    def _rank(self):
        return self.spec.rank or DEFAULT_RANK

    def in_tensors(self):
        s, p = self.spec, self.spec.prefix
        hk, hv = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        return [TensorSpec(f"{p}.q", (hk, s.hidden_size)), TensorSpec(f"{p}.k", (hk, s.hidden_size)),
                TensorSpec(f"{p}.v", (hv, s.hidden_size)), TensorSpec(f"{p}.g", (hv, s.hidden_size)),
                TensorSpec(f"{p}.a1", (s.rank, s.hidden_size), random_shape=(self._rank(), s.hidden_size))]

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def other_tensors(self):
        s, p = self.spec, self.spec.prefix
        hk = s.num_heads * s.key_dim
        return [TensorSpec(f"{p}.a2", (hk, s.rank), random_shape=(hk, self._rank())),
                TensorSpec(f"{p}.a2.b", (hk,), init="normal:2.0"),  # random weights: slow and fast channels
                TensorSpec(f"{p}.norm", (s.value_dim,), init="gain")]

    def bind_others(self, tensors, runtime) -> None:
        p = self.spec.prefix
        self.a2 = take(tensors, f"{p}.a2").contiguous()
        self.a2_bias = take(tensors, f"{p}.a2.b").contiguous()
        self.gain = take(tensors, f"{p}.norm").contiguous()

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        shape = (s.num_heads, s.key_dim, s.value_dim)
        x = ws.get("gla.x", (n, ops.gla_row_width(*shape)), torch.float32)
        raw = ws.get("gla.raw", (n, s.num_heads * s.value_dim), torch.float32)
        ops.gla_prepare(proj, col0, self.a2, self.a2_bias, s.tau, x, n, *shape)
        # single tokens walk the recurrence as it is written; prompt portions take sixteen tokens at a time
        pairs = None
        if ctx.host.max_q_len > 1:
            pairs = ws.get("gla.chunks", (ops.gla_chunks_scratch(n, ctx.n_seqs, *shape),), torch.float32)
        ops.gla_scan(x, cache.tensor, raw, ctx.q_start, cache.slots, ctx.n_seqs, *shape, s.key_dim ** -0.5,
                     chunks=pairs, max_tokens=ctx.host.max_q_len)
        ops.gla_finish(raw, x, self.gain, s.norm_eps, scale, o, n, *shape)


class Retention(BranchMixer):
    """Linear attention with one fixed decay per head: S <- decay_h S + k v^T, o = S^T q, no softmax and no denominator.
    Queries and keys are turned by position, the keys then scaled by key_dim^-1/2; every head's o is divided by its
    root mean square and multiplied by silu(G h). The state is float32 [heads, key_dim, value_dim] per request. The
    recurrence runs on the kernels of gated linear attention, whose rows [q | k | log decay | v | g] a kernel of its
    own prepares; single tokens multiply the state by the decay as the configuration gives it, prompt portions walk
    sixteen tokens at a time by the exponentials of multiples of its logarithm."""

    role = "ret"

    def __init__(self, spec: RetentionSpec):
        if not (0 < spec.key_dim <= ops.GLA_MAX_KEY_HEAD and 0 < spec.value_dim <= ops.GLA_MAX_VALUE_HEAD):
            raise ValueError(f"retention: head sizes {spec.key_dim} / {spec.value_dim} are outside "
                             f"1..{ops.GLA_MAX_KEY_HEAD} / 1..{ops.GLA_MAX_VALUE_HEAD}")
        if spec.num_heads <= 0 or len(spec.decay) != spec.num_heads or not all(0.0 < float(d) <= 1.0 for d in spec.decay):
            raise ValueError("retention: one decay in (0, 1] per head")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.position = make_part("position", spec.position)
        self.neighbours = getattr(spec.position, "pairing", "halves") == "neighbours"
        self.decay = self.log_decay = None

    def cache_spec(self):
        s = self.spec
        return StateCacheSpec((s.num_heads, s.key_dim, s.value_dim), "float32")

    def in_tensors(self):
        s, p = self.spec, self.spec.prefix
        hk, hv = s.num_heads * s.key_dim, s.num_heads * s.value_dim
        return [TensorSpec(f"{p}.q", (hk, s.hidden_size)), TensorSpec(f"{p}.k", (hk, s.hidden_size)),
                TensorSpec(f"{p}.v", (hv, s.hidden_size)), TensorSpec(f"{p}.g", (hv, s.hidden_size))]

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def bind_others(self, tensors, runtime) -> None:
        d = [float(x) for x in self.spec.decay]
        self.decay = torch.tensor(d, dtype=torch.float32, device=runtime.device)
        # the logarithm of the decay as float32 holds it, formed in float64 and rounded once
        self.log_decay = torch.tensor([math.log(float(x)) for x in self.decay.double().tolist()], dtype=torch.float32,
                                      device=runtime.device)

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        shape = (s.num_heads, s.key_dim, s.value_dim)
        x = ws.get("ret.x", (n, ops.gla_row_width(*shape)), torch.float32)
        raw = ws.get("ret.raw", (n, s.num_heads * s.value_dim), torch.float32)
        cos, sin, rot = self.position.rotary(ctx.runtime)
        ops.retention_prepare(proj, col0, self.log_decay, cos, sin, rot, self.neighbours, ctx.positions,
                              s.key_dim ** -0.5, x, n, *shape)
        pairs = None
        if ctx.host.max_q_len > 1:
            pairs = ws.get("ret.chunks", (ops.gla_chunks_scratch(n, ctx.n_seqs, *shape),), torch.float32)
        ops.gla_scan(x, cache.tensor, raw, ctx.q_start, cache.slots, ctx.n_seqs, *shape, 1.0, chunks=pairs,
                     max_tokens=ctx.host.max_q_len, decay=self.decay)
        ops.gla_finish(raw, x, None, s.norm_eps, scale, o, n, *shape)
