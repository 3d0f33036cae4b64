"""Rotary positions as tables of cos and sin by absolute position.

The table is the reference's (`pyre/model.py:41-51`): inv_freq[j] = 1 / theta^(2j/d)
in float32, angle = position * inv_freq[j], cos and sin of it, kept in float32 (the
reference then rounds the table to the model's element type; here the rotation is
done in float32 and only its result is rounded). The halves of the reference's
table repeat each other, so one half is stored.
"""

from __future__ import annotations

import math

import torch

from pyre_amd.parts.base import NoPositionSpec, PositionEncoding, RotarySpec


def scaled_frequencies(inv: torch.Tensor, rotary_dim: int, theta: float, scaling: tuple) -> tuple[torch.Tensor, float]:
    """The frequencies ``inv`` (float64, one per pair) stretched for contexts beyond the ``original`` one, and the factor
    on cosines and sines. With d(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), the index of the pair that turns
    t times over ``original`` positions: pairs up to lo = floor(d(fast)) keep their frequency, pairs from
    hi = ceil(d(slow)) on have it divided by ``factor``, those between are blended linearly by their index."""
    factor, original, fast, slow = (float(x) for x in scaling)

    def index_of(turns: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), rotary_dim - 1)
    ramp = ((torch.arange(inv.numel(), dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return inv / factor * ramp + inv * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotary_tables(rotary_dim: int, theta: float, n_positions: int, exact: bool = False,
                  scaling: tuple | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """cos, sin of shape [n_positions, rotary_dim / 2], float32, on the CPU. ``exact``: the angles are formed in
    float64 and only their cosines and sines are rounded. ``scaling`` (always exact): see :func:`scaled_frequencies`."""
    if exact or scaling is not None:
        inv = theta ** (-torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim)
        mag = 1.0
        if scaling is not None:
            inv, mag = scaled_frequencies(inv, rotary_dim, theta, scaling)
        freqs = torch.outer(torch.arange(n_positions, dtype=torch.float64), inv)
        return (freqs.cos() * mag).float(), (freqs.sin() * mag).float()
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(n_positions, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos(), freqs.sin()


class RotaryEncoding(PositionEncoding):
    def __init__(self, spec: RotarySpec):
        self.spec = spec
        self.rotary_dim = spec.rotary_dim if spec.rotary_dim is not None else spec.head_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= spec.head_dim):
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {spec.head_dim}")
        self._tables = None

    def rotary(self, runtime):
        n = runtime.max_positions  # the engine's longest request decides, as the reference's table grows on demand
        if self._tables is None or self._tables[0].shape[0] < n or self._tables[0].device != runtime.device:
            cos, sin = rotary_tables(self.rotary_dim, self.spec.theta, n, self.spec.exact, getattr(self.spec, "scaling", None))
            self._tables = (cos.to(runtime.device).contiguous(), sin.to(runtime.device).contiguous())
        return self._tables[0], self._tables[1], self.rotary_dim


class NoPosition(PositionEncoding):
    def __init__(self, spec: NoPositionSpec):
        self.spec = spec
