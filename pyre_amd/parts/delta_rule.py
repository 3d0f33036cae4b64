"""The gated delta rule: a float32 matrix state per head and request that every token decays per key channel, corrects
towards its value along its key and reads with its query."""

from __future__ import annotations

import torch

from pyre_amd.hip import ops
from pyre_amd.parts.base import GatedDeltaRuleSpec, StateCacheSpec, TensorSpec, take
from pyre_amd.parts.branch import BranchMixer

#: columns of the two low-rank products that the random-weights mode draws when a description leaves them to the file
DEFAULT_RANK = 8


class GatedDeltaRule(BranchMixer):
    """q, k, v <- silu(conv over time(W h)); q, k unit vectors per head, q times key_dim^-1/2; per value head
    S <- diag(a) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with beta = sigmoid(B h) and
    a = exp(-exp(A_log) softplus(A2 (A1 h) + dt_bias)) per key channel; o / rms(o) * gain * sigmoid(G2 (G1 h)); then the
    output matrix. All its input matrices (B, A1 and G1 among them) are one product.

    Keeps two states per request: S float32 [heads, value_dim, key_dim] (column by column) and the last ``taps - 1`` projected rows of q, k
    and v, which the convolution of the next step's first tokens reads."""

    role = "gdr"

    def __init__(self, spec: GatedDeltaRuleSpec):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError("gated delta rule: heads must be a multiple of kv_heads")
        if not (0 < spec.key_dim <= ops.GDR_MAX_HEAD and 0 < spec.value_dim <= ops.GDR_MAX_HEAD):
            raise ValueError(f"gated delta rule: head sizes {spec.key_dim} / {spec.value_dim} are outside 1..{ops.GDR_MAX_HEAD}")
        if not (1 <= spec.conv_taps <= ops.CONV_MAX_TAPS):
            raise ValueError(f"gated delta rule: {spec.conv_taps} taps are outside 1..{ops.CONV_MAX_TAPS}")
        for r in (spec.decay_rank, spec.gate_rank):
            if r is not None and not (0 < r <= ops.GDR_MAX_RANK):
                raise ValueError(f"gated delta rule: rank {r} is outside 1..{ops.GDR_MAX_RANK}")
        self.spec = spec
        self.hidden_size = spec.hidden_size
        self.inner = spec.num_heads * spec.value_dim
        self.channels = 2 * spec.num_kv_heads * spec.key_dim + spec.num_heads * spec.value_dim
        self.taps = self.a2 = self.g2 = self.dt_bias = self.rate = self.gain = None

    def cache_spec(self):
        s = self.spec
        # a head's state S [key_dim, value_dim] column by column: the rows of a column lie together for the kernel
        return StateCacheSpec((s.num_heads, s.value_dim, s.key_dim), "float32")

    def cache_specs(self) -> list:
        specs = [self.cache_spec()]
        if self.spec.conv_taps > 1:
            specs.append(StateCacheSpec((self.spec.conv_taps - 1, self.channels), "float32"))
        return specs

    def _sizes(self):
        s = self.spec
        return s.num_kv_heads * s.key_dim, s.num_heads * s.key_dim, s.num_heads * s.value_dim

    def in_tensors(self):
        s, p = self.spec, self.spec.prefix
        gk, hk, hv = self._sizes()
        return [TensorSpec(f"{p}.q", (gk, s.hidden_size)), TensorSpec(f"{p}.k", (gk, s.hidden_size)),
                TensorSpec(f"{p}.v", (hv, s.hidden_size)), TensorSpec(f"{p}.b", (s.num_heads, s.hidden_size)),
                TensorSpec(f"{p}.a1", (s.decay_rank, s.hidden_size), random_shape=(s.decay_rank or DEFAULT_RANK, s.hidden_size)),
                TensorSpec(f"{p}.g1", (s.gate_rank, s.hidden_size), random_shape=(s.gate_rank or DEFAULT_RANK, s.hidden_size))]

    def out_tensor(self):
        return TensorSpec(f"{self.spec.prefix}.o", (self.spec.hidden_size, self.inner))

    def other_tensors(self):
        s, p = self.spec, self.spec.prefix
        gk, hk, hv = self._sizes()
        # random weights: taps of the order of one, so that every tap matters; slow and fast channels
        return [TensorSpec(f"{p}.q.conv", (gk, s.conv_taps), init="normal:0.5"),
                TensorSpec(f"{p}.k.conv", (gk, s.conv_taps), init="normal:0.5"),
                TensorSpec(f"{p}.v.conv", (hv, s.conv_taps), init="normal:0.5"),
                TensorSpec(f"{p}.a2", (hk, s.decay_rank), random_shape=(hk, s.decay_rank or DEFAULT_RANK)),
                TensorSpec(f"{p}.g2", (hv, s.gate_rank), random_shape=(hv, s.gate_rank or DEFAULT_RANK)),
                TensorSpec(f"{p}.dt_bias", (hk,), init="normal:1.0"), TensorSpec(f"{p}.A_log", (s.num_heads,), init="normal:1.0"),
                TensorSpec(f"{p}.norm", (s.value_dim,), init="gain")]

    def bind_others(self, tensors, runtime) -> None:
        p = self.spec.prefix
        # [taps, channels]: a tap's weights of neighbouring channels lie together
        self.taps = torch.cat([take(tensors, f"{p}.{x}.conv").float() for x in ("q", "k", "v")], dim=0).t().contiguous()
        self.a2 = take(tensors, f"{p}.a2").contiguous()
        self.g2 = take(tensors, f"{p}.g2").contiguous()
        self.dt_bias = take(tensors, f"{p}.dt_bias").float().contiguous()
        # the factor on the step size, -exp(A_log), one per head, in float32 whatever the file's type
        self.rate = (-torch.exp(take(tensors, f"{p}.A_log").float())).contiguous()
        self.gain = take(tensors, f"{p}.norm").contiguous()

    def attend(self, ctx, proj, col0, cache, o, scale) -> None:
        s, n, ws = self.spec, ctx.n_tokens, ctx.workspace
        state, conv = (cache[0], cache[1]) if isinstance(cache, (list, tuple)) else (cache, None)
        shape = (s.num_heads, s.num_kv_heads, s.key_dim, s.value_dim)
        x = ws.get("gdr.x", (n, ops.gdr_row_width(*shape)), torch.float32)
        raw = ws.get("gdr.raw", (n, s.num_heads * s.value_dim), torch.float32)
        ops.gdr_prepare(proj, col0, self.taps, conv.tensor if conv is not None else None, ctx.state_slots,
                        ctx.seq_of_token, ctx.q_start, ctx.n_seqs, self.a2, self.dt_bias, self.rate, self.g2, s.unit_eps,
                        x, n, *shape)
        ops.gdr_scan(x, state.tensor, raw, ctx.q_start, state.slots, ctx.n_seqs, *shape, max_tokens=ctx.host.max_q_len)
        ops.gdr_finish(raw, x, self.gain, s.norm_eps, scale, o, n, *shape)
