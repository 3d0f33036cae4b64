"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), no biases (`pyre/model.py:128-139`)."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts import fast
from pyre_amd.parts.base import ClippedGLUSpec, FeedForward, GeluGLUSpec, ReluSquaredMLPSpec, SwiGLUSpec, TensorSpec, take
from pyre_amd.parts.linear import Linear, linear_specs


class SwiGLU(FeedForward):
    """gate and up are one product over [Wgate; Wup]; the SiLU-gate reads its halves."""

    def __init__(self, spec: SwiGLUSpec):
        self.spec = spec
        self.gate_up = Linear(spec.hidden_size, 2 * spec.intermediate_size, "ffn.gate_up")
        self.down = Linear(spec.intermediate_size, spec.hidden_size, "ffn.down")

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return (linear_specs(f"{p}.gate_proj", s.intermediate_size, s.hidden_size, False)
                + linear_specs(f"{p}.up_proj", s.intermediate_size, s.hidden_size, False)
                + linear_specs(f"{p}.down_proj", s.hidden_size, s.intermediate_size, False))

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        halves = [take(tensors, f"{p}.gate_proj.weight"), take(tensors, f"{p}.up_proj.weight")]
        fused = torch.cat(halves, dim=0)
        del halves  # the two weights are free before the next layer makes its copy
        self.gate_up.set(fused)
        self.down.set(take(tensors, f"{p}.down_proj.weight"))

    def linears(self) -> list:
        return [self.gate_up, self.down]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        act = ctx.workspace.get("ffn.act", (n, self.spec.intermediate_size), ctx.dtype)
        if not fast.gate_up_silu(self.gate_up, ctx, h, n, act):
            gu = self.gate_up.forward(ctx, h, n)
            ops.silu_mul(gu, act, n)
        return self.down.forward(ctx, act, n)


class ClippedGLU(FeedForward):
    """down(g * sigmoid(slope * g) * (u + 1)) with g = min(gate(x), limit), u = clamp(up(x), -limit, limit):
    a gated unit whose inputs are clipped and whose linear half is shifted by one. gate and up are one
    product over [Wgate; Wup]."""

    def __init__(self, spec: ClippedGLUSpec):
        self.spec = spec
        self.gate_up = Linear(spec.hidden_size, 2 * spec.intermediate_size, "ffn.gate_up")
        self.down = Linear(spec.intermediate_size, spec.hidden_size, "glu.down")

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return [TensorSpec(f"{p}.gate", (s.intermediate_size, s.hidden_size)),
                TensorSpec(f"{p}.up", (s.intermediate_size, s.hidden_size)),
                TensorSpec(f"{p}.down", (s.hidden_size, s.intermediate_size))]

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        halves = [take(tensors, f"{p}.gate"), take(tensors, f"{p}.up")]
        fused = torch.cat(halves, dim=0)
        del halves
        self.gate_up.set(fused)
        self.down.set(take(tensors, f"{p}.down"))

    def linears(self) -> list:
        return [self.gate_up, self.down]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        act = ctx.workspace.get("ffn.act", (n, self.spec.intermediate_size), ctx.dtype)
        # a step of few rows finishes the unit in the gate/up product's epilogue, as the SiLU-gate is finished
        if not fast.gate_up_silu(self.gate_up, ctx, h, n, act, unit=(self.spec.limit, self.spec.slope, 1.0)):
            gu = self.gate_up.forward(ctx, h, n)
            ops.clipped_glu(gu, act, n, self.spec.limit, self.spec.slope)
        return self.down.forward(ctx, act, n)


class GeluGLU(FeedForward):
    """down(gelu_tanh(gate(x)) * up(x)): the gated unit g sigmoid(slope (g + cubic g^3)) u, which is the tanh form of
    GELU on the gate since (1 + tanh z) / 2 = sigmoid(2 z). gate and up are one product over [Wgate; Wup]; a step of
    few rows finishes the unit in that product's epilogue."""

    UNIT = (0.0, ops.GELU_TANH_SLOPE, 0.0, ops.GELU_TANH_CUBIC)  #: no clipping, no shift

    def __init__(self, spec: GeluGLUSpec):
        self.spec = spec
        self.gate_up = Linear(spec.hidden_size, 2 * spec.intermediate_size, "ffn.gate_up")
        self.down = Linear(spec.intermediate_size, spec.hidden_size, "geglu.down")

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return [TensorSpec(f"{p}.gate", (s.intermediate_size, s.hidden_size)),
                TensorSpec(f"{p}.up", (s.intermediate_size, s.hidden_size)),
                TensorSpec(f"{p}.down", (s.hidden_size, s.intermediate_size))]

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        halves = [take(tensors, f"{p}.gate"), take(tensors, f"{p}.up")]
        fused = torch.cat(halves, dim=0)
        del halves
        self.gate_up.set(fused)
        self.down.set(take(tensors, f"{p}.down"))

    def linears(self) -> list:
        return [self.gate_up, self.down]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        act = ctx.workspace.get("ffn.act", (n, self.spec.intermediate_size), ctx.dtype)
        if not fast.gate_up_silu(self.gate_up, ctx, h, n, act, unit=self.UNIT):
            gu = self.gate_up.forward(ctx, h, n)
            limit, slope, shift, cubic = self.UNIT
            ops.clipped_glu(gu, act, n, limit, slope, shift, cubic)
        return self.down.forward(ctx, act, n)


class ReluSquaredMLP(FeedForward):
    """down(relu(up(x))^2): no gate, the activation is the square of the positive part."""

    def __init__(self, spec: ReluSquaredMLPSpec):
        self.spec = spec
        self.up = Linear(spec.hidden_size, spec.intermediate_size, "relu2.up")
        self.down = Linear(spec.intermediate_size, spec.hidden_size, "relu2.down")

    def tensor_specs(self) -> list[TensorSpec]:
        s, p = self.spec, self.spec.prefix
        return [TensorSpec(f"{p}.up", (s.intermediate_size, s.hidden_size)),
                TensorSpec(f"{p}.down", (s.hidden_size, s.intermediate_size))]

    def bind(self, tensors, runtime) -> None:
        p = self.spec.prefix
        self.up.set(take(tensors, f"{p}.up"))
        self.down.set(take(tensors, f"{p}.down"))

    def linears(self) -> list:
        return [self.up, self.down]

    def forward(self, ctx, h):
        n = ctx.n_tokens
        act = ctx.workspace.get("ffn.act", (n, self.spec.intermediate_size), ctx.dtype)
        ops.relu2(self.up.forward(ctx, h, n), act, n)
        return self.down.forward(ctx, act, n)
