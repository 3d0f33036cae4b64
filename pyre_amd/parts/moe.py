"""A mixture of small feed-forward layers with a sigmoid router and a shared expert."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.base import FeedForward, GroupedSoftmaxMoESpec, SigmoidMoESpec, SoftmaxTopKMoESpec, TensorSpec, take
from pyre_amd.parts.linear import Linear


class SigmoidMoE(FeedForward):
    """out = sum over the chosen experts e of w_e down_e(relu(up_e h)^2) + the shared expert's result.

    The router's logits are a product of their own (float32 sums); a kernel squashes them, chooses and writes the
    weights as a dense row per token, zero where an expert is not chosen. All experts' ways up (and the shared
    one's behind them) are one product over the row-wise concatenation of their matrices; the activation kernel
    squares, weights and zeroes; all ways down are one product over the column-wise concatenation, which sums the
    weighted results and the shared expert's as it goes. Every token streams through every expert's matrices:
    right for steps whose tokens between them choose most experts anyway."""

    def __init__(self, spec: SigmoidMoESpec):
        if not (0 < spec.top <= spec.experts <= ops.ROUTE_MAX_EXPERTS):
            raise ValueError(f"mixture: {spec.top} of {spec.experts} experts is not a choice the routing kernel makes")
        if spec.expert_size <= 0 or spec.shared_size < 0:
            raise ValueError("mixture: bad expert sizes")
        self.spec = spec
        self.inner = spec.experts * spec.expert_size + spec.shared_size
        self.router = Linear(spec.hidden_size, spec.experts, "moe.router")
        self.up = Linear(spec.hidden_size, self.inner, "moe.up")
        self.down = Linear(self.inner, spec.hidden_size, "moe.down")

    def _experts(self) -> list[str]:
        s = self.spec
        return [f"{s.prefix}.e{i}" for i in range(s.experts)] + ([f"{s.prefix}.shared"] if s.shared_size else [])

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(f"{s.prefix}.router", (s.experts, s.hidden_size))]
        for p in self._experts():
            ff = s.shared_size if p.endswith(".shared") else s.expert_size
            specs += [TensorSpec(f"{p}.up", (ff, s.hidden_size)), TensorSpec(f"{p}.down", (s.hidden_size, ff))]
        return specs

    def bind(self, tensors, runtime) -> None:
        s = self.spec
        self.router.set(take(tensors, f"{s.prefix}.router"))
        ups = [take(tensors, f"{p}.up") for p in self._experts()]
        self.up.set(torch.cat(ups, dim=0))
        del ups
        downs = [take(tensors, f"{p}.down") for p in self._experts()]
        self.down.set(torch.cat(downs, dim=1))
        del downs

    def linears(self) -> list:
        return [self.router, self.up, self.down]

    def forward(self, ctx, h):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        gates = ws.get("moe.gates", (n, s.experts), torch.float32)
        ops.route_topk(self.router.forward(ctx, h, n), gates, n, s.top)
        act = ws.get("moe.act", (n, self.inner), ctx.dtype)
        ops.expert_act(self.up.forward(ctx, h, n), gates, act, n, s.experts, s.expert_size, s.shared_size)
        return self.down.forward(ctx, act, n)


class GroupedSoftmaxMoE(FeedForward):
    """out = sum over the chosen experts e of s_e f_e(h): s = softmax(router h) over experts and identity experts alike;
    the choice goes by s + correction among the experts of the best groups; f_e = down_e(silu(gate_e h) * (up_e h)) for
    an expert with matrices, f_e(h) = h for an identity expert.

    The router's logits are a product of their own (float32 sums); one kernel makes the softmax, the groups' choice and
    the experts' and writes a dense row of weights per token. All experts' gates and ways up are one product over
    [G_0; ..; G_E-1; U_0; ..; U_E-1], the activation kernel gates, weights and zeroes, all ways down are one product over
    [D_0 | .. | D_E-1], which sums the weighted results as it goes; the identity experts' share, (sum of their weights)
    h, is added to that product's first partial sum. Every token streams through every expert's matrices."""

    def __init__(self, spec: GroupedSoftmaxMoESpec):
        total = spec.experts + spec.identity
        if spec.experts <= 0 or spec.identity < 0 or total > ops.ROUTE_MAX_EXPERTS:
            raise ValueError(f"mixture: {spec.experts} + {spec.identity} experts are not a number the routing kernel takes")
        if spec.groups <= 0 or total % spec.groups or not (0 < spec.keep_groups <= spec.groups):
            raise ValueError(f"mixture: {total} experts do not form {spec.groups} equal groups, or {spec.keep_groups} "
                             "of them cannot be kept")
        if not (0 < spec.top <= spec.keep_groups * (total // spec.groups)):
            raise ValueError(f"mixture: {spec.top} experts cannot be chosen from {spec.keep_groups} groups of "
                             f"{total // spec.groups}")
        if spec.expert_size <= 0:
            raise ValueError("mixture: bad expert size")
        self.spec = spec
        self.total = total
        self.inner = spec.experts * spec.expert_size
        self.router = Linear(spec.hidden_size, total, "gmoe.router")
        self.gate_up = Linear(spec.hidden_size, 2 * self.inner, "gmoe.gate_up")
        self.down = Linear(self.inner, spec.hidden_size, "gmoe.down")
        self.correction = None

    def _experts(self) -> list[str]:
        return [f"{self.spec.prefix}.e{i}" for i in range(self.spec.experts)]

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(f"{s.prefix}.router", (self.total, s.hidden_size)),
                 TensorSpec(f"{s.prefix}.correction", (self.total,), init="normal:0.1")]
        for p in self._experts():
            specs += [TensorSpec(f"{p}.gate", (s.expert_size, s.hidden_size)), TensorSpec(f"{p}.up", (s.expert_size, s.hidden_size)),
                      TensorSpec(f"{p}.down", (s.hidden_size, s.expert_size))]
        return specs

    def bind(self, tensors, runtime) -> None:
        s = self.spec
        self.router.set(take(tensors, f"{s.prefix}.router"))
        self.correction = take(tensors, f"{s.prefix}.correction").float().contiguous()
        parts = [take(tensors, f"{p}.gate") for p in self._experts()] + [take(tensors, f"{p}.up") for p in self._experts()]
        self.gate_up.set(torch.cat(parts, dim=0))
        del parts
        downs = [take(tensors, f"{p}.down") for p in self._experts()]
        self.down.set(torch.cat(downs, dim=1))
        del downs

    def linears(self) -> list:
        return [self.router, self.gate_up, self.down]

    def forward(self, ctx, h):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        gates = ws.get("gmoe.gates", (n, self.total), torch.float32)
        ops.route_grouped(self.router.forward(ctx, h, n), self.correction, gates, n, s.top, s.groups, s.keep_groups)
        act = ws.get("gmoe.act", (n, self.inner), ctx.dtype)
        ops.expert_glu_act(self.gate_up.forward(ctx, h, n), gates, act, n, s.experts, s.expert_size)
        out = self.down.forward(ctx, act, n)
        if s.identity:
            if out.data.dtype != torch.float32 or out.bias is not None:  # a product that hands on rounded sums: summed first
                full = ws.get("gmoe.sum", (1, n, s.hidden_size), torch.float32)
                ops.reduce_partials(out, full[0], n)
                out = type(out)(full)
            ops.add_weighted_rows(out, h, gates, s.experts, s.identity, n)
        return out


class SoftmaxTopKMoE(FeedForward):
    """out = sum over the chosen experts e of w_e down_e(silu(gate_e h) * (up_e h)) + g down_s(silu(gate_s h) * (up_s h)):
    the ``top`` experts of largest router logit z = R h + b, their weights the softmax over the chosen logits alone; the
    shared expert s runs for every token, times g = sigmoid(sg . h).

    The router's logits are a product of their own (float32 sums) whose last row is the shared expert's gate; one kernel
    chooses, takes the softmax and writes a dense row of weights per token, the gate's sigmoid behind them. All experts'
    gates and ways up, the shared one's behind them, are one product over [G_0; ..; G_E-1; G_s; U_0; ..; U_E-1; U_s], the
    activation kernel gates, weights and zeroes, all ways down are one product over [D_0 | .. | D_E-1 | D_s], which sums
    the weighted results as it goes. Every token streams through every expert's matrices."""

    def __init__(self, spec: SoftmaxTopKMoESpec):
        if not (0 < spec.top <= spec.experts <= ops.ROUTE_MAX_EXPERTS):
            raise ValueError(f"mixture: {spec.top} of {spec.experts} experts is not a choice the routing kernel makes")
        if spec.expert_size <= 0 or spec.shared_size < 0:
            raise ValueError("mixture: bad expert sizes")
        self.spec = spec
        self.extra = 1 if spec.shared_size and spec.shared_gate else 0
        self.inner = spec.experts * spec.expert_size + spec.shared_size
        self.router = Linear(spec.hidden_size, spec.experts + self.extra, "stmoe.router")
        self.gate_up = Linear(spec.hidden_size, 2 * self.inner, "stmoe.gate_up")
        self.down = Linear(self.inner, spec.hidden_size, "stmoe.down")

    def _experts(self) -> list[tuple[str, int]]:
        s = self.spec
        return [(f"{s.prefix}.e{i}", s.expert_size) for i in range(s.experts)] + \
               ([(f"{s.prefix}.shared", s.shared_size)] if s.shared_size else [])

    def tensor_specs(self) -> list[TensorSpec]:
        s = self.spec
        specs = [TensorSpec(f"{s.prefix}.router", (s.experts, s.hidden_size))]
        if s.router_bias:
            specs.append(TensorSpec(f"{s.prefix}.router.b", (s.experts,)))
        for p, ff in self._experts():
            specs += [TensorSpec(f"{p}.gate", (ff, s.hidden_size)), TensorSpec(f"{p}.up", (ff, s.hidden_size)),
                      TensorSpec(f"{p}.down", (s.hidden_size, ff))]
        if self.extra:
            specs.append(TensorSpec(f"{s.prefix}.shared.sg", (1, s.hidden_size)))
        return specs

    def bind(self, tensors, runtime) -> None:
        s = self.spec
        rows = [take(tensors, f"{s.prefix}.router")]
        if self.extra:
            rows.append(take(tensors, f"{s.prefix}.shared.sg").to(rows[0].dtype))
        bias = None
        if s.router_bias:
            bias = take(tensors, f"{s.prefix}.router.b").float()
            if self.extra:
                bias = torch.cat([bias, torch.zeros(self.extra, dtype=torch.float32, device=bias.device)])
        self.router.set(torch.cat(rows, dim=0) if len(rows) > 1 else rows[0], bias)
        del rows
        parts = [take(tensors, f"{p}.gate") for p, _ in self._experts()] + [take(tensors, f"{p}.up") for p, _ in self._experts()]
        self.gate_up.set(torch.cat(parts, dim=0))
        del parts
        downs = [take(tensors, f"{p}.down") for p, _ in self._experts()]
        self.down.set(torch.cat(downs, dim=1))
        del downs

    def linears(self) -> list:
        return [self.router, self.gate_up, self.down]

    def forward(self, ctx, h):
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        gates = ws.get("stmoe.gates", (n, s.experts + self.extra), torch.float32)
        ops.route_topk(self.router.forward(ctx, h, n), gates, n, s.top, softmax=True, extra=self.extra)
        act = ws.get("stmoe.act", (n, self.inner), ctx.dtype)
        ops.expert_glu_act(self.gate_up.forward(ctx, h, n), gates, act, n, s.experts, s.expert_size, s.shared_size,
                           s.experts if self.extra else -1)
        return self.down.forward(ctx, act, n)
