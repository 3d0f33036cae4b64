"""RMSNorm fused with the residual sum that precedes it (`pyre/model.py:22-38,151-152`)."""

from __future__ import annotations

from pyre_amd.hip import ops
from pyre_amd.parts.base import LayerNormSpec, Norm, RMSNormSpec, TanhNormSpec, TensorSpec, take


class RMSNorm(Norm):
    def __init__(self, spec: RMSNormSpec):
        self.spec = spec
        self.gain = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.tensor, (self.spec.hidden_size,), init="normal:0.1" if self.spec.one_plus else "gain")]

    def bind(self, tensors, runtime) -> None:
        self.gain = tensors[self.spec.tensor].contiguous()
        if self.spec.one_plus:
            # a weight stored around zero: the gain is one plus it, formed in float32 whatever the file's type
            self.gain = (1.0 + self.gain.float()).contiguous()

    def forward(self, ctx, resid, delta, out, rows=None) -> None:
        if delta is not None and (delta.post is not None or delta.more is not None or delta.outer is not None
                                  or delta.scale != 1.0):
            # a pending term that is normed or scaled before it is added, or comes with another
            ops.add_rms_terms(resid, delta, self.gain, self.spec.eps, out, rows)
            return
        ops.add_rmsnorm(resid, delta, self.gain, self.spec.eps, out, rows)


class LayerNorm(Norm):
    """(x - mean) / sqrt(var + eps) * gain without a bias, fused with the residual sum before it. The
    pending term may carry a norm of its own (``Partials.post``: a sublayer's result that is normed
    and scaled before it is added); the same kernel applies it."""

    def __init__(self, spec: LayerNormSpec):
        self.spec = spec
        self.gain = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.spec.name, (self.spec.hidden_size,), init="gain")]

    def bind(self, tensors, runtime) -> None:
        self.gain = tensors[self.spec.name].contiguous()

    def forward(self, ctx, resid, delta, out, rows=None) -> None:
        ops.add_layernorm(resid, delta, self.gain, self.spec.eps, out, rows)


class TanhNorm(Norm):
    """tanh(alpha x) * gain + shift with one learned number alpha: no mean, no variance, so a row is normed
    element by element. Fused with the residual sum before it; takes up to two pending terms, each with a factor
    (``Partials.scale``, ``Partials.more``)."""

    def __init__(self, spec: TanhNormSpec):
        self.spec = spec
        self.gain = self.shift = self.alpha = None

    def tensor_specs(self) -> list[TensorSpec]:
        n, h = self.spec.name, self.spec.hidden_size
        # random weights: alpha one, so that rows of unit scale use the bend of the tanh
        return [TensorSpec(n, (h,), init="gain"), TensorSpec(f"{n}.b", (h,), init="normal"),
                TensorSpec(f"{n}.alpha", (), init="gain")]

    def bind(self, tensors, runtime) -> None:
        n = self.spec.name
        self.gain = take(tensors, n).contiguous()
        self.shift = take(tensors, f"{n}.b").to(self.gain.dtype).contiguous()
        self.alpha = take(tensors, f"{n}.alpha").to(self.gain.dtype).reshape(1).contiguous()

    def forward(self, ctx, resid, delta, out, rows=None) -> None:
        ops.add_tanhnorm(resid, delta, self.alpha, self.gain, self.shift, out, rows)
