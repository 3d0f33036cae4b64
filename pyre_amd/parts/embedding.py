"""Token embedding (`pyre/model.py:162,196`) and output head (`:172,201`)."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.base import BigramEmbeddingSpec, EmbeddingSpec, LMHeadSpec, Part, StateCacheSpec, TensorSpec
from pyre_amd.parts.linear import Linear


class TokenEmbedding(Part):
    def __init__(self, spec: EmbeddingSpec):
        self.spec = spec
        self.table = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.vocab_size, self.spec.hidden_size))]

    def bind(self, tensors, runtime) -> None:
        self.table = tensors[self.spec.name].contiguous()

    def forward(self, ctx, resid: torch.Tensor) -> None:
        """resid[n] = float32(table[token n]) * scale: the residual stream starts here."""
        ops.embed(self.table, ctx.tokens, resid, self.spec.scale)


class BigramEmbedding(Part):
    """table[token] + pairs[row of (previous token, token)]: a second table indexed by a hash of the pair, whose last
    row is for a request's first token. The previous token of the first token that a request brings in a step is state
    that the request keeps on the device (one float32 whose value is the token's number, exact below 2^24), so a step
    whose tokens are results still on the device needs nothing from the host."""

    def __init__(self, spec: BigramEmbeddingSpec):
        if spec.buckets <= 0 or spec.mul_prev < 0 or spec.mul_cur < 0:
            raise ValueError("bigram embedding: buckets must be positive, the multipliers not negative")
        if spec.buckets >= 1 << 31:
            raise ValueError("bigram embedding: more buckets than a 32-bit row number holds")
        if spec.vocab_size >= 1 << 24:
            raise ValueError("bigram embedding: the previous token is kept as a float32, which holds numbers below 2^24")
        self.spec = spec
        self.table = self.pairs = None

    def cache_specs(self) -> list:
        return [StateCacheSpec((1,), "float32")]

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        return [TensorSpec(s.name, (s.vocab_size, s.hidden_size)), TensorSpec(s.pairs_name, (s.buckets + 1, s.hidden_size))]

    def bind(self, tensors, runtime) -> None:
        self.table = tensors[self.spec.name].contiguous()
        self.pairs = tensors[self.spec.pairs_name].to(self.table.dtype).contiguous()

    def forward(self, ctx, resid: torch.Tensor, caches: list) -> None:
        s = self.spec
        # (p a + t b) mod m = (p (a mod m) + t (b mod m)) mod m: the kernel's 64-bit products hold whatever the multipliers are
        ops.bigram_embed(self.table, self.pairs, ctx.tokens, ctx.positions, ctx.seq_of_token, ctx.q_start,
                         caches[0].tensor, caches[0].slots, resid, s.buckets, s.mul_prev % s.buckets, s.mul_cur % s.buckets)


class LMHead(Part):
    """logits = h W^T in float32, for the wanted rows only. A tied head shares the
    embedding's memory (the reference copies it, `pyre/loader.py:58-61`)."""

    def __init__(self, spec: LMHeadSpec):
        self.spec = spec
        self.linear = Linear(spec.hidden_size, spec.vocab_size, "head")

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.vocab_size, self.spec.hidden_size),
                           alias_of=self.spec.tied_to)]

    def bind(self, tensors, runtime) -> None:
        self.linear.set(tensors[self.spec.name])

    def linears(self) -> list:
        return [self.linear]

    def forward(self, ctx, h: torch.Tensor, m: int) -> torch.Tensor:
        out = ctx.workspace.get("head.logits", (m, self.spec.vocab_size), torch.float32)
        p = self.linear.forward(ctx, h, m, out=out)
        if p.data.data_ptr() != out.data_ptr() or p.count != 1 or p.bias is not None:
            ops.reduce_partials(p, out, m)
        if self.spec.scale != 1.0:
            ops.scale_(out, self.spec.scale)
        if self.spec.softcap:
            ops.softcap_(out, self.spec.softcap)
        return out
