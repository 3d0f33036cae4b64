"""A layer's input from the token itself: a slice of a second token table, gated by a narrow product of the stream."""

from __future__ import annotations

from pyre_amd.hip import ops
from pyre_amd.parts.base import Part, TensorSpec, TokenSideSpec, take
from pyre_amd.parts.linear import Linear


class TokenSide(Part):
    """y = proj(gelu_tanh(gate x) * table[token, first : first + dim]): x the rows of the residual stream, the table one
    for all layers, each of which takes its own columns. The step's tokens are read on the device, so a step whose
    tokens are results still on their way needs nothing from the host."""

    def __init__(self, spec: TokenSideSpec):
        if spec.dim <= 0 or spec.first < 0 or spec.first + spec.dim > spec.table_width:
            raise ValueError(f"token side: columns {spec.first}..{spec.first + spec.dim} lie outside the table's "
                             f"{spec.table_width}")
        self.spec = spec
        self.gate = Linear(spec.hidden_size, spec.dim, "side.gate")
        self.proj = Linear(spec.dim, spec.hidden_size, "side.proj")
        self.table = None

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        return [TensorSpec(s.table, (s.vocab_size, s.table_width)), TensorSpec(f"{s.prefix}.gate", (s.dim, s.hidden_size)),
                TensorSpec(f"{s.prefix}.proj", (s.hidden_size, s.dim))]

    def bind(self, tensors, runtime) -> None:
        s = self.spec
        self.table = take(tensors, s.table).contiguous()
        self.gate.set(take(tensors, f"{s.prefix}.gate"))
        self.proj.set(take(tensors, f"{s.prefix}.proj"))

    def linears(self) -> list:
        return [self.gate, self.proj]

    def forward(self, ctx, h):
        s, n = self.spec, ctx.n_tokens
        g = ctx.workspace.get("side.g", (n, s.dim), ctx.dtype)
        ops.token_side_gate(self.gate.forward(ctx, h, n), self.table, s.first, ctx.tokens, g, n)
        return self.proj.forward(ctx, g, n)
