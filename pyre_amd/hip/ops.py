"""The kernels as functions of torch tensors.

torch is the allocator and the owner of the stream here, nothing more: every
function checks shapes, element types, device and contiguity on the host, then
hands raw pointers to the HIP library. There is no CPU path; a tensor that is
not on a GPU is an error.
"""

from __future__ import annotations

from dataclasses import dataclass
from functools import lru_cache

import torch

from pyre_amd.hip.lib import KernelError, call

_DT = {torch.float32: 0, torch.bfloat16: 1}


def dtype_code(t: torch.Tensor | torch.dtype) -> int:
    dt = t if isinstance(t, torch.dtype) else t.dtype
    try:
        return _DT[dt]
    except KeyError:
        raise KernelError(f"unsupported element type {dt}; kernels take float32 and bfloat16") from None


_STREAM: int | None = None


def use_stream(handle: int | None) -> None:
    """Put every kernel on this HIP stream until told otherwise (None: ask torch for its
    current stream at every call again). A step asks once instead of once per kernel."""
    global _STREAM
    _STREAM = handle


def _stream() -> int:
    return _STREAM if _STREAM is not None else torch.cuda.current_stream().cuda_stream


def _dev(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operand is not on a GPU (there is no CPU path)")


def _contig(name: str, t: torch.Tensor) -> None:
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")


def _i32(name: str, t: torch.Tensor, n: int | None = None) -> None:
    if t.dtype != torch.int32:
        raise KernelError(f"{name} must be int32, got {t.dtype}")
    _contig(name, t)
    if n is not None and t.numel() < n:
        raise KernelError(f"{name} holds {t.numel()} entries, {n} needed")


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


@dataclass
class PostNorm:
    """The norm of a sublayer's own result: LN(term; eps) * gain (* scale), element by element (``kind`` "layer"),
    or term / sqrt(mean(term^2) + eps) * gain (``kind`` "rms")."""

    gain: torch.Tensor
    eps: float
    scale: torch.Tensor | None = None
    kind: str = "layer"


@dataclass
class Partials:
    """What a matrix product hands to its consumer: ``S`` partial sums ``[S, M, N]``
    (``S`` = 1 unless the product was split along K) and a bias not yet added.
    The consumer adds them up in the order 0..S-1, then the bias."""

    data: torch.Tensor
    bias: torch.Tensor | None = None
    #: a norm (and layer scale) that the term goes through before it is added: only a norm
    #: that says so takes such a term (:func:`add_layernorm`)
    post: "PostNorm | None" = None
    #: a factor on the whole term (sums and bias), and another term to be added with it (a layer whose
    #: mixer and feed-forward read the same rows hands on both): only a norm that says so takes them
    scale: float = 1.0
    more: "Partials | None" = None
    #: a norm that the sum of this term and of ``more`` (each after its own norm and factor) goes through before it is
    #: added: only a norm that says so takes it (:func:`add_rms_terms`)
    outer: "PostNorm | None" = None

    def __post_init__(self) -> None:
        if self.data.dim() != 3 or not self.data.is_contiguous():
            raise KernelError("partials must be a contiguous [S, M, N] tensor")

    @property
    def count(self) -> int:
        return self.data.shape[0]

    @property
    def rows(self) -> int:
        return self.data.shape[1]

    @property
    def width(self) -> int:
        return self.data.shape[2]

    @property
    def stride(self) -> int:
        return self.data.stride(0)

    def _args(self, width: int):
        if self.width != width:
            raise KernelError(f"partials are {self.width} wide, {width} expected")
        if self.bias is not None and self.bias.numel() != width:
            raise KernelError(f"bias has {self.bias.numel()} entries, {width} expected")
        return (self.data.data_ptr(), dtype_code(self.data), self.count, self.stride,
                _ptr(self.bias), dtype_code(self.bias) if self.bias is not None else 0)


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> None:
    """out[n] = float32(table[ids[n]]) * scale; ids must already be checked against the vocabulary."""
    _dev(table, ids, out)
    n, hidden = out.shape
    if table.dim() != 2 or table.shape[1] != hidden or out.dtype != torch.float32:
        raise KernelError("embed: table [V, H] and float32 out [N, H] expected")
    _contig("table", table), _contig("out", out), _i32("ids", ids, n)
    call("pyre_embed", table.data_ptr(), dtype_code(table), ids.data_ptr(), out.data_ptr(), n, hidden,
         float(scale), _stream())


def add_rmsnorm(resid: torch.Tensor, delta: Partials | None, gain: torch.Tensor, eps: float,
                out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """resid += delta (all partials, then bias); out = rmsnorm(resid) * gain.

    With ``rows`` only those rows are normed, into ``out[0:len(rows)]``, and
    ``resid`` is left as it was.
    """
    _dev(resid, gain, out, rows)
    hidden = resid.shape[-1]
    if resid.dtype != torch.float32 or resid.dim() != 2:
        raise KernelError("add_rmsnorm: the residual stream is float32 [N, H]")
    n = resid.shape[0] if rows is None else rows.numel()
    if out.shape[-1] != hidden or out.shape[0] < n or gain.numel() != hidden:
        raise KernelError("add_rmsnorm: shapes of out / gain do not fit the residual")
    _contig("resid", resid), _contig("out", out), _contig("gain", gain)
    if rows is not None:
        _i32("rows", rows)
    if delta is not None:
        if delta.rows < resid.shape[0]:
            raise KernelError("add_rmsnorm: delta has fewer rows than the residual")
        if delta.post is not None or delta.scale != 1.0 or delta.more is not None or delta.outer is not None:
            raise KernelError("add_rmsnorm: a term that is normed or scaled before it is added, or comes with another, is not taken")
        d = delta._args(hidden)
    else:
        d = (None, 0, 0, 0, None, 0)
    call("pyre_add_rmsnorm", resid.data_ptr(), *d, gain.data_ptr(), dtype_code(gain), out.data_ptr(),
         dtype_code(out), _ptr(rows), n, hidden, float(eps), _stream())


def add_layernorm(resid: torch.Tensor, delta: Partials | None, gain: torch.Tensor, eps: float,
                  out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """resid += y; out = LN(resid) * gain, with LN(x) = (x - mean) / sqrt(var + eps) and y the
    pending term (all partials, then bias), which goes through its own norm first if it carries one
    (``delta.post``: y = LN(term; post.eps) * post.gain * post.scale).

    With ``rows`` only those rows are normed, into ``out[0:len(rows)]``, and ``resid`` is left as it was.
    """
    _dev(resid, gain, out, rows)
    hidden = resid.shape[-1]
    if resid.dtype != torch.float32 or resid.dim() != 2:
        raise KernelError("add_layernorm: the residual stream is float32 [N, H]")
    n = resid.shape[0] if rows is None else rows.numel()
    if out.shape[-1] != hidden or out.shape[0] < n or gain.numel() != hidden:
        raise KernelError("add_layernorm: shapes of out / gain do not fit the residual")
    _contig("resid", resid), _contig("out", out), _contig("gain", gain)
    if rows is not None:
        _i32("rows", rows)
    post = (None, 0, None, 0, 0.0)
    if delta is not None:
        if delta.rows < resid.shape[0]:
            raise KernelError("add_layernorm: delta has fewer rows than the residual")
        if delta.scale != 1.0 or delta.more is not None or delta.outer is not None or \
                (delta.post is not None and delta.post.kind != "layer"):
            raise KernelError("add_layernorm: a term that is scaled before it is added, or comes with another, is not taken")
        d = delta._args(hidden)
        if delta.post is not None:
            pn = delta.post
            _dev(pn.gain, pn.scale)
            if pn.gain.numel() != hidden or (pn.scale is not None and pn.scale.numel() != hidden):
                raise KernelError("add_layernorm: the pending term's gain / scale do not fit the residual")
            _contig("post.gain", pn.gain)
            if pn.scale is not None:
                _contig("post.scale", pn.scale)
            post = (pn.gain.data_ptr(), dtype_code(pn.gain), _ptr(pn.scale),
                    dtype_code(pn.scale) if pn.scale is not None else 0, float(pn.eps))
    else:
        d = (None, 0, 0, 0, None, 0)
    call("pyre_add_layernorm", resid.data_ptr(), *d, *post, gain.data_ptr(), dtype_code(gain), out.data_ptr(),
         dtype_code(out), _ptr(rows), n, hidden, float(eps), _stream())


#: slope and cubic term that make g sigmoid(slope (g + cubic g^3)) the tanh form of GELU: (1 + tanh z) / 2 = sigmoid(2 z)
GELU_TANH_SLOPE, GELU_TANH_CUBIC = 2.0 * (2.0 / 3.141592653589793) ** 0.5, 0.044715


def clipped_glu(gu: Partials, out: torch.Tensor, n: int, limit: float, slope: float, shift: float = 1.0,
                cubic: float = 0.0) -> None:
    """out[n, i] = g * sigmoid(slope * (g + cubic g^3)) * (u + shift) with g = min(gate, limit),
    u = clamp(up, -limit, limit), gate = gu[:, :I], up = gu[:, I:] (``limit`` <= 0: no clipping)."""
    _dev(gu.data, out)
    inter = out.shape[-1]
    if gu.width != 2 * inter or gu.rows < n or out.shape[0] < n:
        raise KernelError("clipped_glu: gate/up buffer does not fit the output")
    if gu.bias is not None:
        raise KernelError("clipped_glu: a pending bias is not supported")
    _contig("out", out)
    call("pyre_clipped_glu", gu.data.data_ptr(), dtype_code(gu.data), gu.count, gu.stride, out.data_ptr(),
         dtype_code(out), n, inter, float(limit), float(slope), float(shift), float(cubic), _stream())


def scale_(x: torch.Tensor, s: float) -> None:
    """x *= s in place (contiguous float32)."""
    _dev(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("scale_: contiguous float32 expected")
    call("pyre_scale", x.data_ptr(), x.numel(), float(s), _stream())


def _proj_args(proj: Partials, col0: int, width: int):
    if proj.bias is not None:
        raise KernelError("a fused input product with a pending bias is not taken")
    if col0 < 0 or col0 + width > proj.width:
        raise KernelError(f"columns {col0}..{col0 + width} lie outside the product's {proj.width}")
    return (proj.data.data_ptr(), dtype_code(proj.data), proj.count, proj.stride, proj.width, col0)


def unit_qkv_write(proj: Partials, col0: int, q_out: torch.Tensor, k_cache: torch.Tensor | None,
                   v_cache: torch.Tensor | None, gate_out: torch.Tensor | None, slots: torch.Tensor | None, n: int,
                   nq: int, nkv: int, dk: int, dv: int, page_size: int, unit_norm: bool, eps: float) -> None:
    """Finish a step's input product from column ``col0`` on (``nq`` query and ``nkv`` key heads of ``dk``,
    ``nkv`` value heads of ``dv``, then ``nq`` gates if ``gate_out`` is given): queries and keys divided by
    their root mean square over ``dk`` (``unit_norm``), queries to ``q_out [N, nq*dk]``, keys and values to
    ``k_cache [pages, nkv, page, dk]`` / ``v_cache [pages, nkv, page, dv]`` at ``slots`` (-1: not stored),
    sigmoid(gate) to float32 ``gate_out [N, nq]``."""
    _dev(proj.data, q_out, k_cache, v_cache, gate_out, slots)
    width = (nq + nkv) * dk + nkv * dv + (nq if gate_out is not None else 0)
    args = _proj_args(proj, col0, width)
    if proj.rows < n or q_out.numel() < n * nq * dk:
        raise KernelError("unit_qkv_write: buffers are smaller than the batch")
    _contig("q_out", q_out)
    write = k_cache is not None
    cache_dt = dtype_code(q_out)
    if write:
        if v_cache is None or slots is None:
            raise KernelError("unit_qkv_write: k cache without v cache or slots")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, dk) or tuple(v_cache.shape[1:]) != (nkv, page_size, dv) \
                or k_cache.dtype != v_cache.dtype:
            raise KernelError(f"unit_qkv_write: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                              f"nkv={nkv} page={page_size} dk={dk} dv={dv}")
        cache_dt = dtype_code(k_cache)
    if gate_out is not None and (gate_out.dtype != torch.float32 or gate_out.numel() < n * nq or not gate_out.is_contiguous()):
        raise KernelError("unit_qkv_write: gates are contiguous float32 [N, nq]")
    call("pyre_unit_qkv_write", *args, q_out.data_ptr(), dtype_code(q_out), _ptr(k_cache), _ptr(v_cache), cache_dt,
         _ptr(gate_out), _ptr(slots), n, nq, nkv, dk, dv, page_size, int(bool(unit_norm)), float(eps),
         1 if write else 0, _stream())


ATTN_BIASED_TILE_MAX_KEY_HEAD = 128  #: the largest key head of the tile kernel (attention_biased.hip)


def _attn_biased_common(q, out, k_cache, v_cache, gate, positions, seq_of_token, block_table, bias, far,
                        nq, nkv, dk, dv, page_size, sink=None, gate_dim=1):
    _dev(q, out, k_cache, v_cache, gate, positions, seq_of_token, block_table, bias, sink)
    if gate_dim not in (1, dv):
        raise KernelError("attn_biased: a gate per head or per element of the value head")
    if sink is not None and (sink.dtype != torch.float32 or not sink.is_contiguous() or sink.numel() != nq):
        raise KernelError(f"attn_biased: the sinks are contiguous float32 [{nq}]")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attn_biased: queries, caches and output share one element type")
    if tuple(k_cache.shape[1:]) != (nkv, page_size, dk) or tuple(v_cache.shape[1:]) != (nkv, page_size, dv):
        raise KernelError("attn_biased: cache shapes do not fit the head geometry")
    _contig("q", q), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
    if out.dim() != 2 or out.stride(1) != 1 or out.shape[1] < nq * dv:
        raise KernelError("attn_biased: out is [N, >= nq*dv] with contiguous rows")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn_biased: block table must be int32 [rows, pages]")
    _i32("positions", positions), _i32("seq_of_token", seq_of_token)
    if gate is not None and (gate.dtype != torch.float32 or not gate.is_contiguous()):
        raise KernelError("attn_biased: gates are contiguous float32 [N, nq] or [N, nq*dv]")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or tuple(bias.shape) != (nq, far + 1)):
        raise KernelError(f"attn_biased: the bias by distance is float32 [{nq}, {far + 1}]")


def attn_biased_tile(q, out, k_cache, v_cache, gate, out_scale, tiles, n_tiles, positions, seq_of_token,
                     block_table, nq, nkv, dk, dv, page_size, scale, cap, bias, far, window, keep_first, chunk: int = 0,
                     sink: torch.Tensor | None = None, gate_dim: int = 1) -> None:
    """Prompt portions of the capped, biased attention; ``tiles`` is int32 [n_tiles, 2] = (first token, count <= 32).
    ``sink`` (float32 [nq]): exp(sink) of the head joins the softmax's denominator, a key without a value.
    ``gate_dim`` = dv: ``gate`` is [N, nq*dv], a gate per element of the output."""
    _attn_biased_common(q, out, k_cache, v_cache, gate, positions, seq_of_token, block_table, bias, far,
                        nq, nkv, dk, dv, page_size, sink, gate_dim)
    _i32("tiles", tiles, 2 * n_tiles)
    call("pyre_attn_biased_tile", q.data_ptr(), out.data_ptr(), out.stride(0), dtype_code(q), k_cache.data_ptr(),
         v_cache.data_ptr(), _ptr(gate), float(out_scale), tiles.data_ptr(), n_tiles, positions.data_ptr(),
         seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0), nq, nkv, dk, dv, page_size,
         float(scale), float(cap), _ptr(bias), int(far), int(window), int(keep_first), int(chunk), _ptr(sink),
         int(gate_dim), _stream())


def attn_biased_spans(table_width: int, page_size: int, window: int, keep_first: int, chunk: int = 0) -> int:
    """Spans of 128 keys that a token can have when its block table is ``table_width`` pages wide."""
    from pyre_amd.hip.lib import lib

    return int(lib().pyre_attn_biased_spans(max(1, table_width * page_size), int(window), int(keep_first), int(chunk)))


def attn_biased_single(q, out, k_cache, v_cache, gate, out_scale, tokens, n, positions, seq_of_token,
                       block_table, nq, nkv, dk, dv, page_size, scale, cap, bias, far, window, keep_first,
                       scratch: torch.Tensor | None = None, chunk: int = 0, sink: torch.Tensor | None = None,
                       gate_dim: int = 1) -> None:
    """The same for ``n`` tokens one by one (``tokens``: which of the flat batch, None: the first n). ``scratch``
    (float32, ``n * nq * attn_biased_spans(...) * (dv + 2)`` elements): a block per span of 128 keys and a second
    kernel that joins them, instead of a block per token and head that takes its spans in turn. ``sink`` and
    ``gate_dim`` as for :func:`attn_biased_tile`."""
    _attn_biased_common(q, out, k_cache, v_cache, gate, positions, seq_of_token, block_table, bias, far,
                        nq, nkv, dk, dv, page_size, sink, gate_dim)
    if tokens is not None:
        _dev(tokens), _i32("tokens", tokens, n)
    spans = 0
    if scratch is not None:
        _dev(scratch)
        spans = attn_biased_spans(block_table.shape[1], page_size, window, keep_first, chunk)
        if scratch.dtype != torch.float32 or not scratch.is_contiguous() or scratch.numel() < n * nq * spans * (dv + 2):
            raise KernelError(f"attn_biased_single: scratch of {n * nq * spans * (dv + 2)} float32 elements needed")
    call("pyre_attn_biased_single", q.data_ptr(), out.data_ptr(), out.stride(0), dtype_code(q), k_cache.data_ptr(),
         v_cache.data_ptr(), _ptr(gate), float(out_scale), _ptr(tokens), n, positions.data_ptr(),
         seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0), nq, nkv, dk, dv, page_size,
         float(scale), float(cap), _ptr(bias), int(far), int(window), int(keep_first), int(chunk), _ptr(scratch), spans,
         _ptr(sink), int(gate_dim), _stream())


GLA_MAX_RANK = 512     #: the widest low-rank input of the decay (linear_attention.hip)
GLA_MAX_KEY_HEAD = 256
GLA_MAX_VALUE_HEAD = 256


def gla_row_width(heads: int, dk: int, dv: int) -> int:
    """Columns of the float32 rows [q | k | log decay | v | g] that the recurrent kernels share."""
    return 3 * heads * dk + 2 * heads * dv


def gla_prepare(proj: Partials, col0: int, a2: torch.Tensor, a2_bias: torch.Tensor | None, tau: float,
                x: torch.Tensor, n: int, heads: int, dk: int, dv: int) -> None:
    """Finish the input product from column ``col0`` on (q, k: heads*dk each; v, g: heads*dv each; then the
    low-rank input of the decay) into float32 rows ``x`` and put log(sigmoid(a2 @ low + bias)) / tau there."""
    _dev(proj.data, a2, a2_bias, x)
    rank = a2.shape[1]
    args = _proj_args(proj, col0, 2 * heads * dk + 2 * heads * dv + rank)
    if tuple(a2.shape) != (heads * dk, rank) or (a2_bias is not None and a2_bias.numel() != heads * dk):
        raise KernelError("gla_prepare: the decay's second matrix is [heads*dk, rank], its bias [heads*dk]")
    _contig("a2", a2)
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[-1] != gla_row_width(heads, dk, dv) or x.shape[0] < n \
            or proj.rows < n:
        raise KernelError("gla_prepare: x is contiguous float32 [>= n, 3*heads*dk + 2*heads*dv]")
    call("pyre_gla_prepare", *args, a2.data_ptr(), dtype_code(a2), _ptr(a2_bias),
         dtype_code(a2_bias) if a2_bias is not None else 0, float(tau), x.data_ptr(), n, heads, dk, dv, rank, _stream())


def gla_chunks_scratch(n_tokens: int, n_seqs: int, heads: int, dk: int, dv: int) -> int:
    """Float32 elements of scratch that the walk in chunks needs for such a step."""
    from pyre_amd.hip.lib import lib

    fn = lib().pyre_gla_chunks_scratch
    fn.restype = __import__("ctypes").c_long
    return int(fn(n_tokens, n_seqs, heads, dk, dv))


def gla_scan(x: torch.Tensor, state: torch.Tensor, o: torch.Tensor, q_start: torch.Tensor, state_slots: torch.Tensor,
             n_seqs: int, heads: int, dk: int, dv: int, qscale: float, chunks: torch.Tensor | None = None,
             max_tokens: int = 0, decay: torch.Tensor | None = None) -> None:
    """The recurrence over each request's tokens of the step, from and into ``state [slots, heads, dk, dv]``;
    ``o`` (float32 [N, heads*dv]) receives qscale * S^T q. ``chunks``: scratch (float32,
    :func:`gla_chunks_scratch` elements) that makes the walk take sixteen tokens at a time on the matrix cores
    (for steps that carry prompt portions, ``max_tokens`` the most that one request brings; the token-by-token
    walk is the one for single tokens): a difference of rounding. ``decay`` (float32 [heads]): the token-by-token walk
    multiplies head h's state by decay[h] itself instead of by the exponential of the rows' logarithms (which must be its
    logarithm all the same: the walk in chunks goes by them)."""
    _dev(x, state, o, q_start, state_slots, chunks, decay)
    if decay is not None and (decay.dtype != torch.float32 or decay.numel() != heads or not decay.is_contiguous()):
        raise KernelError("gla_scan: one float32 decay per head")
    for name, t in (("x", x), ("state", state), ("o", o)):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError(f"gla_scan: {name} is contiguous float32")
    if tuple(state.shape[1:]) != (heads, dk, dv) or x.shape[-1] != gla_row_width(heads, dk, dv) or o.shape[-1] != heads * dv:
        raise KernelError("gla_scan: shapes do not fit the head geometry")
    _i32("q_start", q_start, n_seqs + 1), _i32("state_slots", state_slots, n_seqs)
    if chunks is None:
        call("pyre_gla_scan", x.data_ptr(), state.data_ptr(), o.data_ptr(), q_start.data_ptr(), state_slots.data_ptr(),
             n_seqs, heads, dk, dv, float(qscale), _ptr(decay), _stream())
        return
    n = o.shape[0]
    if chunks.dtype != torch.float32 or not chunks.is_contiguous() or chunks.numel() < gla_chunks_scratch(n, n_seqs, heads, dk, dv):
        raise KernelError("gla_scan: the chunks' scratch is contiguous float32 of gla_chunks_scratch(...) elements")
    call("pyre_gla_chunks", x.data_ptr(), chunks.data_ptr(), state.data_ptr(), o.data_ptr(), q_start.data_ptr(),
         state_slots.data_ptr(), n, n_seqs, int(max_tokens), heads, dk, dv, float(qscale), _stream())


def gla_finish(o: torch.Tensor, x: torch.Tensor, gain: torch.Tensor | None, eps: float, out_scale: float, out: torch.Tensor,
               n: int, heads: int, dk: int, dv: int) -> None:
    """out[n, h*dv + e] = o / rms(o over dv) * gain[e] * silu(g) * out_scale (``gain`` None: ones); ``out`` has contiguous rows."""
    _dev(o, x, gain, out)
    if o.dtype != torch.float32 or x.dtype != torch.float32 or not o.is_contiguous() or not x.is_contiguous():
        raise KernelError("gla_finish: o and x are contiguous float32")
    if (gain is not None and gain.numel() != dv) or out.dim() != 2 or out.stride(1) != 1 or out.shape[1] < heads * dv or out.shape[0] < n:
        raise KernelError("gla_finish: gain [dv] and out [>= n, >= heads*dv] expected")
    if gain is not None:
        _contig("gain", gain)
    call("pyre_gla_finish", o.data_ptr(), x.data_ptr(), _ptr(gain), dtype_code(gain) if gain is not None else 0, float(eps), float(out_scale),
         out.data_ptr(), dtype_code(out), out.stride(0), n, heads, dk, dv, _stream())


def rope_kv_write(qkv: Partials, q_out: torch.Tensor, k_cache: torch.Tensor | None,
                  v_cache: torch.Tensor | None, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  rotary_dim: int, positions: torch.Tensor, slots: torch.Tensor | None, n: int,
                  nq: int, nkv: int, hd: int, page_size: int) -> None:
    """Finish the q/k/v projection (partials + bias), rotate q and k by position,
    store q in ``q_out [N, nq*hd]`` and, when a cache is given, k and v in their pages.

    ``k_cache`` is one layer's ``[pages, nkv, page_size, hd]``; ``v_cache`` the same
    layer's ``[pages, nkv, hd, page_size]``. ``slots[n] = page * page_size + offset``,
    or -1 for a token that is not to be stored.
    """
    _dev(qkv.data, q_out, k_cache, v_cache, cos, sin, positions, slots)
    width = (nq + 2 * nkv) * hd
    q = qkv._args(width)
    if qkv.rows < n or q_out.numel() < n * nq * hd:
        raise KernelError("rope_kv_write: buffers are smaller than the batch")
    _contig("q_out", q_out), _i32("positions", positions, n)
    write = k_cache is not None
    cache_dt = 0
    if write:
        if v_cache is None or slots is None:
            raise KernelError("rope_kv_write: k cache without v cache or slots")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
            raise KernelError(f"rope_kv_write: cache shapes {tuple(k_cache.shape)} / {tuple(v_cache.shape)} "
                              f"do not fit nkv={nkv} page={page_size} hd={hd}")
        cache_dt = dtype_code(k_cache)
    if rotary_dim:
        if cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32:
            raise KernelError("rope_kv_write: float32 cos/sin tables needed")
        if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or cos.shape != sin.shape:
            raise KernelError("rope_kv_write: cos/sin tables must be [positions, rotary_dim/2]")
        _contig("cos", cos), _contig("sin", sin)
    call("pyre_rope_kv_write", *q, q_out.data_ptr(), dtype_code(q_out), _ptr(k_cache), _ptr(v_cache),
         cache_dt, _ptr(cos), _ptr(sin), rotary_dim, positions.data_ptr(), _ptr(slots), n, nq, nkv, hd,
         page_size, 1 if write else 0, _stream())


def silu_mul(gu: Partials, out: torch.Tensor, n: int) -> None:
    """out[n, i] = silu(gate[n, i]) * up[n, i] with gate = gu[:, :I], up = gu[:, I:]."""
    _dev(gu.data, out)
    inter = out.shape[-1]
    if gu.width != 2 * inter or gu.rows < n or out.shape[0] < n:
        raise KernelError("silu_mul: gate/up buffer does not fit the output")
    if gu.bias is not None:
        raise KernelError("silu_mul: a pending bias is not supported")
    _contig("out", out)
    call("pyre_silu_mul", gu.data.data_ptr(), dtype_code(gu.data), gu.count, gu.stride, out.data_ptr(),
         dtype_code(out), n, inter, _stream())


def reduce_partials(p: Partials, out: torch.Tensor, n: int) -> None:
    _dev(p.data, out)
    if out.shape[-1] != p.width or out.shape[0] < n or p.rows < n:
        raise KernelError("reduce_partials: shapes do not fit")
    _contig("out", out)
    call("pyre_reduce_partials", *p._args(p.width), out.data_ptr(), dtype_code(out), n, p.width, _stream())


_FILL_PATTERNS = {(4, "zero"): 0, (2, "zero"): 0, (4, "nan"): 0x7FC00000, (2, "nan"): 0x7FC0}


def fill_rows(tensor: torch.Tensor, ids: list[int], value: float) -> None:
    """tensor[:, id] = value for every listed id; ``tensor`` is contiguous ``[outer, rows, ...]``
    of float32 or bfloat16, ``value`` is 0.0 or NaN (state slots are zeroed with it, freed pages
    poisoned)."""
    import ctypes
    import math

    _dev(tensor)
    _contig("tensor", tensor)
    if tensor.dim() < 2 or tensor.dtype not in _DT:
        raise KernelError("fill_rows: a float32 or bfloat16 tensor [outer, rows, ...] expected")
    if not ids:
        return
    kind = "nan" if math.isnan(value) else "zero" if value == 0.0 else None
    if kind is None:
        raise KernelError("fill_rows: the value must be 0 or NaN")
    outer, rows = tensor.shape[0], tensor.shape[1]
    row_elems = tensor.stride(1)
    arr = (ctypes.c_int * len(ids))(*[int(i) for i in ids])
    with torch.cuda.device(tensor.device):
        call("pyre_fill_rows", tensor.data_ptr(), tensor.element_size(), tensor.stride(0), outer, rows, row_elems,
             ctypes.cast(arr, ctypes.c_void_p), len(ids), _FILL_PATTERNS[(tensor.element_size(), kind)], _stream())


def gemm_generic(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor,
                 m: int, a_rows: torch.Tensor | None = None) -> None:
    """out[0:m] = a[0:m] (or a[a_rows]) @ w.T (+ bias), fp32 accumulation in ascending k."""
    _dev(a, w, bias, out, a_rows)
    n_out, k = w.shape
    if a.dim() != 2 or a.shape[1] != k or out.dim() != 2 or out.shape[1] != n_out:
        raise KernelError(f"gemm: a {tuple(a.shape)} @ w {tuple(w.shape)}.T -> out {tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    if out.shape[0] < m or (a_rows is None and a.shape[0] < m):
        raise KernelError("gemm: fewer rows than m")
    if a_rows is not None:
        _i32("a_rows", a_rows, m)
    if bias is not None and bias.numel() != n_out:
        raise KernelError("gemm: bias length")
    call("pyre_gemm_generic", a.data_ptr(), dtype_code(a), a.stride(0), _ptr(a_rows), w.data_ptr(),
         dtype_code(w), w.stride(0), _ptr(bias), dtype_code(bias) if bias is not None else 0,
         out.data_ptr(), dtype_code(out), out.stride(0), m, n_out, k, _stream())


F32_KSPLIT_MAX = 8

#: compute units that launch plans are made for when nobody names a device (an MI355X)
DEFAULT_UNITS = 256


def compute_units(device=None) -> int:
    """Compute units of ``device`` (torch's current one if None), as the kernel library sees
    them: its kernels that fill the chip in one round of blocks go by the same number."""
    from pyre_amd.hip.lib import lib

    if device is None:
        return int(lib().pyre_compute_units())
    with torch.cuda.device(device):
        return int(lib().pyre_compute_units())


def gemm_f32_ksplit(n_out: int, k: int, units: int = DEFAULT_UNITS) -> int:
    """Into how many parts of k the float32 product is split: enough blocks of 128 output
    columns for the ``units`` compute units, parts of at least 512. A function of the weight's
    shape (and the engine's device) alone, never of the rows, so that a row's result does not
    depend on its step."""
    blocks = -(-n_out // 128)
    return max(1, min(F32_KSPLIT_MAX, units // blocks, k // 512))


def gemm_f32(a: torch.Tensor, w: torch.Tensor, bias: torch.Tensor | None, out: torch.Tensor, m: int,
             ksplit: int = 1) -> None:
    """out[0:m] = a[0:m] @ w.T (+ bias) with float32 operands and result, on the matrix cores'
    float32 instruction; the order of an element's additions depends on k alone. With
    ``ksplit`` > 1, ``out`` is [ksplit, m, N]: partial sums over parts of k (the bias in part 0)."""
    _dev(a, w, bias, out)
    n_out, k = w.shape
    if a.dtype != torch.float32 or w.dtype != torch.float32 or out.dtype != torch.float32:
        raise KernelError("gemm_f32: float32 operands and result expected")
    if a.dim() != 2 or a.shape[1] != k or out.shape[-1] != n_out or out.dim() != (2 if ksplit == 1 else 3):
        raise KernelError(f"gemm_f32: a {tuple(a.shape)} @ w {tuple(w.shape)}.T -> out {tuple(out.shape)} do not fit")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(-1) != 1:
        raise KernelError("gemm_f32: rows must be contiguous")
    if out.shape[-2] < m or a.shape[0] < m or (ksplit > 1 and (out.shape[0] != ksplit or out.shape[1] != m)):
        raise KernelError("gemm_f32: fewer rows than m, or partial sums that are not [ksplit, m, N]")
    if bias is not None and bias.numel() != n_out:
        raise KernelError("gemm_f32: bias length")
    call("pyre_gemm_f32", a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), _ptr(bias),
         dtype_code(bias) if bias is not None else 0, out.data_ptr(), out.stride(-2),
         out.stride(0) if ksplit > 1 else 0, m, n_out, k, ksplit, _stream())


def attn_generic(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 positions: torch.Tensor, seq_of_token: torch.Tensor, block_table: torch.Tensor,
                 n: int, nq: int, nkv: int, hd: int, page_size: int, scale: float,
                 window: int = 0, tokens: torch.Tensor | None = None,
                 scratch: torch.Tensor | None = None, matrix_cores: bool = True) -> None:
    """Causal attention of n tokens over the paged cache (``tokens``: which of the flat batch,
    else the first n); see attention_generic.hip. ``scratch``: float32 memory of
    ``attn_generic_scratch(...)`` elements for the partial results of the spans of keys; without
    it the memory is allocated here when the block table is wider than one span. ``matrix_cores``:
    float32 queries and caches with a head size of 16, 32, ..., 128 and pages of a multiple of 16
    tokens go to the kernel that serves the query heads of a key/value head from one read of its
    keys and values, on the matrix cores' float32 instruction (its sums run in another order than
    those of one block per head, which False asks for: a difference of rounding)."""
    _dev(q, out, k_cache, v_cache, positions, seq_of_token, block_table, tokens, scratch)
    if q.dtype != out.dtype or q.numel() < n * nq * hd or out.numel() < n * nq * hd:
        raise KernelError("attn: q/out buffers do not fit")
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn: cache shapes do not fit the head geometry")
    if k_cache.dtype != v_cache.dtype:
        raise KernelError("attn: k and v caches differ in element type")
    _contig("q", q), _contig("out", out), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
    _i32("positions", positions, n), _i32("seq_of_token", seq_of_token, n)
    if tokens is not None:
        _i32("tokens", tokens, n)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn: block table must be int32 [rows, pages]")
    max_keys = _attn_generic_keys(block_table.shape[1], page_size, window)
    need = attn_generic_scratch(n, nq, hd, block_table.shape[1], page_size, window)
    if need and scratch is None:
        scratch = torch.empty(need, dtype=torch.float32, device=q.device)
    if need and (scratch.dtype != torch.float32 or not scratch.is_contiguous() or scratch.numel() < need):
        raise KernelError(f"attn: scratch of {need} float32 elements needed")
    per_launch = _attn_generic_rows(n, nq, hd, max_keys)
    flat_q, flat_out = q.view(-1), out.view(-1)
    for at in range(0, n, per_launch):
        rows = min(per_launch, n - at)
        if tokens is not None:  # the list moves on; q, out and positions are indexed by its entries
            args = (flat_q, flat_out, tokens[at:], positions, seq_of_token)
        else:
            args = (flat_q[at * nq * hd:], flat_out[at * nq * hd:], None, positions[at:], seq_of_token[at:])
        call("pyre_attn_generic", args[0].data_ptr(), args[1].data_ptr(), dtype_code(q), k_cache.data_ptr(),
             v_cache.data_ptr(), dtype_code(k_cache), _ptr(args[2]), args[3].data_ptr(), args[4].data_ptr(),
             block_table.data_ptr(), block_table.stride(0), rows, nq, nkv, hd, page_size, float(scale),
             int(window), max_keys, _ptr(scratch) if need else None, int(bool(matrix_cores)), _stream())


ATTN_GENERIC_SCRATCH = 1 << 25   #: float32 elements of scratch that one launch of attn_generic may use
#: the largest head that any attention kernel takes (attention_generic.hip's kMaxHead: a block of
#: 256 threads holds one element each) and the most query heads of a launch (a grid dimension)
ATTN_MAX_HEAD_DIM = 256
ATTN_MAX_HEADS = 65535


def _attn_generic_keys(table_width: int, page_size: int, window: int) -> int:
    """No token sees more keys than its block table holds, or than its window."""
    keys = max(1, table_width * page_size)
    return min(keys, window) if window > 0 else keys


def _attn_generic_rows(n: int, nq: int, hd: int, max_keys: int) -> int:
    """Tokens to a launch: all of them, or as many as the scratch of one launch allows."""
    from pyre_amd.hip.lib import lib

    spans = int(lib().pyre_attn_generic_spans(max_keys))
    return n if spans <= 1 else max(1, min(n, ATTN_GENERIC_SCRATCH // (nq * spans * (hd + 2))))


def attn_generic_scratch(n: int, nq: int, hd: int, table_width: int, page_size: int, window: int = 0) -> int:
    """Float32 elements of scratch that ``attn_generic`` needs for such a call (0: none)."""
    from pyre_amd.hip.lib import lib

    max_keys = _attn_generic_keys(table_width, page_size, window)
    spans = int(lib().pyre_attn_generic_spans(max_keys))
    return 0 if spans <= 1 or n <= 0 else _attn_generic_rows(n, nq, hd, max_keys) * nq * spans * (hd + 2)


def attn_prefill_f32(q, out, k_cache, v_cache, tiles, n_tiles, positions, seq_of_token, block_table,
                     nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions in true float32 on the matrix cores; ``tiles`` is int32
    [n_tiles, 2] = (first token, count <= 32)."""
    _dev(q, out, k_cache, v_cache, tiles, positions, seq_of_token, block_table)
    for name, t in (("q", q), ("out", out), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.dtype != torch.float32:
            raise KernelError(f"attn_prefill_f32: {name} must be float32")
        _contig(name, t)
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn_prefill_f32: cache shapes do not fit the head geometry")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn_prefill_f32: block table must be int32 [rows, pages]")
    _i32("positions", positions), _i32("seq_of_token", seq_of_token), _i32("tiles", tiles, 2 * n_tiles)
    call("pyre_attn_prefill_f32", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         tiles.data_ptr(), n_tiles, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), nq, nkv, hd, page_size, float(scale), int(window), _stream())


ARGMAX_SCRATCH_PER_ROW = 128  #: 4-byte words of scratch per row of logits


def argmax(logits: torch.Tensor, out: torch.Tensor, scratch: torch.Tensor | None = None) -> None:
    """out[i] = index of the largest logit of row i (the lowest index among equals).
    ``scratch``: int32 or float32 device memory of 128 words per row (allocated if absent)."""
    _dev(logits, out, scratch)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: float32 [M, V] logits expected")
    m = logits.shape[0]
    _i32("out", out, m)
    if scratch is None:
        scratch = torch.empty(m * ARGMAX_SCRATCH_PER_ROW, dtype=torch.int32, device=logits.device)
    if scratch.element_size() != 4 or scratch.numel() < m * ARGMAX_SCRATCH_PER_ROW or not scratch.is_contiguous():
        raise KernelError("argmax: scratch must hold 128 four-byte words per row")
    call("pyre_argmax", logits.data_ptr(), logits.stride(0), out.data_ptr(), scratch.data_ptr(), m,
         logits.shape[1], _stream())


ARGMAX_STATIC_MAX_ROWS = 256  #: rows that the library's built-in scratch holds


def argmax_static_init(device=None) -> None:
    """Look the built-in scratch's address up on ``device`` (torch's current one if None). The
    first :func:`argmax_static` on a device does this by itself, which must not happen while a
    stream is capturing: whoever captures calls this beforehand."""
    if device is None:
        call("pyre_argmax_static_init")
    else:
        with torch.cuda.device(device):
            call("pyre_argmax_static_init")


def argmax_static(logits: torch.Tensor, out: torch.Tensor) -> None:
    """:func:`argmax` for callers that must not allocate: the partial results go to an
    array inside the library's device image (at most 256 rows; calls that overlap on one
    GPU race)."""
    _dev(logits, out)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax: float32 [M, V] logits expected")
    m = logits.shape[0]
    _i32("out", out, m)
    with torch.cuda.device(logits.device):
        call("pyre_argmax_static", logits.data_ptr(), logits.stride(0), out.data_ptr(), m, logits.shape[1],
             _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor) -> None:
    """Rows with temperature > 0 get a token drawn by inverse CDF with their
    uniform number; rows with temperature <= 0 keep what ``out`` holds."""
    _dev(logits, temperature, uniform, out)
    m = logits.shape[0]
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample: float32 [M, V] logits expected")
    for name, t in (("temperature", temperature), ("uniform", uniform)):
        if t.dtype != torch.float32 or t.numel() < m or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be contiguous float32 [M]")
    _i32("out", out, m)
    call("pyre_sample", logits.data_ptr(), logits.stride(0), temperature.data_ptr(), uniform.data_ptr(),
         out.data_ptr(), m, logits.shape[1], _stream())


def feed_tokens(tokens: torch.Tensor, src: torch.Tensor, ids: torch.Tensor, n: int) -> None:
    """tokens[i] = ids[src[i]] for i < n with src[i] >= 0 (all int32 on the device)."""
    _dev(tokens, src, ids)
    _i32("tokens", tokens, n), _i32("src", src, n), _i32("ids", ids)
    call("pyre_feed_tokens", tokens.data_ptr(), src.data_ptr(), ids.data_ptr(), n, _stream())


@lru_cache(maxsize=4096)
def attn_mfma_supports(hd: int, page_size: int, nq: int, nkv: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_attn_mfma_supports(hd, page_size, nq, nkv))


def _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size):
    _dev(q, out, k_cache, v_cache, positions, seq_of_token, block_table)
    for name, t in (("q", q), ("out", out), ("k_cache", k_cache), ("v_cache", v_cache)):
        if t.dtype != torch.bfloat16:
            raise KernelError(f"attn (MFMA): {name} must be bfloat16")
        _contig(name, t)
    if tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
        raise KernelError("attn (MFMA): cache shapes do not fit the head geometry")
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise KernelError("attn (MFMA): block table must be int32 [rows, pages]")
    _i32("positions", positions), _i32("seq_of_token", seq_of_token)


def attn_decode_work_bf16(q, out, k_cache, v_cache, work, capacity, positions, seq_of_token, block_table,
                          part_acc, part_ml, counters, alone, nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of single new tokens over the paged cache from a work list (int32
    ``[1 + blocks, 8]``: see ``pyre_attn_decode_work_bf16`` in pyre_api.h) in a launch of
    ``capacity`` blocks per key/value head, one (``alone``) or two to a compute unit.
    ``counters`` must be zero and is left at zero."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("work", work, 8 * (1 + capacity))
    items = nkv * -(-(nq // nkv) // 16)
    if part_acc.dtype != torch.float32 or part_acc.numel() < capacity * items * 16 * hd:
        raise KernelError("attn_decode_work: partial accumulators too small")
    if part_ml.dtype != torch.float32 or part_ml.numel() < capacity * items * 32:
        raise KernelError("attn_decode_work: partial max/sum buffer too small")
    if counters.dtype != torch.int32 or counters.numel() < capacity * items:
        raise KernelError("attn_decode_work: too few counters")
    call("pyre_attn_decode_work_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), capacity, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), part_acc.data_ptr(), part_ml.data_ptr(), counters.data_ptr(), int(bool(alone)), nq,
         nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def attn_decode_work_rope_supports(hd: int, page_size: int, nq: int, nkv: int, partial_stride: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_attn_decode_work_rope_supports(hd, page_size, nq, nkv, partial_stride))


def attn_decode_work_rope_bf16(qkv: Partials, cos, sin, slots, out, k_cache, v_cache, write_kv, work, capacity,
                               positions, seq_of_token, block_table, part_acc, part_ml, counters, alone, nq, nkv, hd,
                               page_size, scale, window=0) -> None:
    """:func:`attn_decode_work_bf16` for a step of single tokens, straight from the step's q/k/v
    product (float32 partial sums and bias): the kernel sums, biases and rotates the queries itself and
    writes each token's rotated key and its value into the cache (``write_kv``) with the arithmetic
    of :func:`rope_kv_write`, the same bits, so that no kernel runs between product and attention.
    ``cos``/``sin``: float32 ``[positions, hd / 2]`` (full-head rotation)."""
    _attn_common(out, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _dev(qkv.data, cos, sin, slots, work, part_acc, part_ml, counters)
    width = (nq + 2 * nkv) * hd
    args = qkv._args(width)
    if qkv.data.dtype != torch.float32:
        raise KernelError("attn_decode_work_rope: float32 partial sums expected")
    if not attn_decode_work_rope_supports(hd, page_size, nq, nkv, qkv.stride):
        raise KernelError(f"attn_decode_work_rope: head_dim {hd}, page_size {page_size}, heads {nq}/{nkv} are not taken")
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.dim() != 2 or cos.shape[1] != hd // 2 \
            or cos.shape != sin.shape:
        raise KernelError("attn_decode_work_rope: float32 cos/sin tables [positions, hd / 2] needed")
    _contig("cos", cos), _contig("sin", sin), _i32("slots", slots, qkv.rows), _i32("work", work, 8 * (1 + capacity))
    items = nkv * -(-(nq // nkv) // 16)
    if part_acc.dtype != torch.float32 or part_acc.numel() < capacity * items * 16 * hd:
        raise KernelError("attn_decode_work: partial accumulators too small")
    if part_ml.dtype != torch.float32 or part_ml.numel() < capacity * items * 32:
        raise KernelError("attn_decode_work: partial max/sum buffer too small")
    if counters.dtype != torch.int32 or counters.numel() < capacity * items:
        raise KernelError("attn_decode_work: too few counters")
    call("pyre_attn_decode_work_rope_bf16", args[0], args[2], args[3], args[4], args[5], cos.data_ptr(), sin.data_ptr(),
         slots.data_ptr(), qkv.rows, int(bool(write_kv)), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), capacity, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), part_acc.data_ptr(), part_ml.data_ptr(), counters.data_ptr(), int(bool(alone)), nq,
         nkv, hd, page_size, float(scale), int(window), _stream())


def attn_prefill_bf16(q, out, k_cache, v_cache, tiles, n_tiles, positions, seq_of_token, block_table,
                      nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions, every wave reading the cache directly; ``tiles`` is int32
    [n_tiles, 2] = (first token, count <= 32)."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("tiles", tiles, 2 * n_tiles)
    call("pyre_attn_prefill_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         tiles.data_ptr(), n_tiles, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
         block_table.stride(0), nq, nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def attn_prefill_waves(nq: int, nkv: int) -> int:
    from pyre_amd.hip.lib import lib

    return int(lib().pyre_attn_prefill_waves(nq, nkv))


def attn_prefill_work_bf16(q, out, k_cache, v_cache, work, n_items, partials, counters, n_slots, positions,
                           seq_of_token, block_table, nq, nkv, hd, page_size, scale, window=0) -> None:
    """Attention of prompt portions for heads of up to 128 elements from a work list (int32
    ``[n_items, 8]``: see ``pyre_attn_prefill_work_bf16`` in pyre_api.h) whose tiles of several
    blocks use the partial slots 0..n_slots-1. ``counters`` must be zero and is left at zero."""
    _attn_common(q, out, k_cache, v_cache, positions, seq_of_token, block_table, nq, nkv, hd, page_size)
    _i32("work", work, 8 * n_items)
    waves = attn_prefill_waves(nq, nkv)
    per_slot = nkv * -(-(nq // nkv) // waves) * waves
    if n_slots:
        if partials.dtype != torch.float32 or partials.numel() < n_slots * per_slot * (hd // 32 * 1024 + 128):
            raise KernelError("attn_prefill_work: partial results do not fit")
        if counters.dtype != torch.int32 or counters.numel() < n_slots * per_slot:
            raise KernelError("attn_prefill_work: too few counters")
    call("pyre_attn_prefill_work_bf16", q.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         work.data_ptr(), n_items, _ptr(partials) if n_slots else None, _ptr(counters) if n_slots else None,
         n_slots, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0),
         nq, nkv, hd, page_size, float(scale), int(window), _stream())


@lru_cache(maxsize=4096)
def gemm_skinny_supports(m: int, n: int, k: int, ldx: int, ldw: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_gemm_skinny_supports(m, n, k, ldx, ldw))


def _skinny_common(x, w, m):
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny: bfloat16 operands expected")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.shape[0] < m:
        raise KernelError(f"gemm_skinny: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit {m} rows")
    if x.stride(1) != 1 or w.stride(1) != 1:
        raise KernelError("gemm_skinny: rows must be contiguous")


def gemm_skinny_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, ksplit: int) -> None:
    """out[s] (float32 [ksplit, m, N]) = partial sums over k of x[0:m] @ w.T, 1 <= m <= 64."""
    _skinny_common(x, w, m)
    n = w.shape[0]
    if out.dtype != torch.float32 or not out.is_contiguous() or out.numel() < ksplit * m * n or not out.is_cuda:
        raise KernelError("gemm_skinny: out must be contiguous float32 [ksplit, m, N] on the GPU")
    call("pyre_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), m, n,
         w.shape[1], ksplit, _stream())


def _gate_shape(unit) -> tuple[float, float, float, float]:
    """(limit, slope, shift, cubic) of the gated unit g sigmoid(slope (g + cubic g^3)) (u + shift); a unit given
    with three numbers has no cubic term."""
    vals = [float(v) for v in unit]
    if len(vals) == 3:
        vals.append(0.0)
    if len(vals) != 4:
        raise KernelError("a gated unit is (limit, slope, shift[, cubic])")
    return tuple(vals)


def gemm_skinny_silu_bf16(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, m: int,
                          unit: tuple[float, float, float] | None = None) -> None:
    """out[0:m] (bfloat16 [m, I]) = silu(x @ gate.T) * (x @ up.T) with w_gate_up = [gate; up]. ``unit`` =
    (limit, slope, shift[, cubic]): g * sigmoid(slope * (g + cubic g^3)) * (u + shift) with g = min(gate, limit),
    u = clamp(up, -limit, limit) instead (limit <= 0: no clipping)."""
    _skinny_common(x, w_gate_up, m)
    two_i = w_gate_up.shape[0]
    if (out.dtype != torch.bfloat16 or not out.is_contiguous() or not out.is_cuda or out.dim() != 2
            or out.shape[1] * 2 != two_i or out.shape[0] < m):
        raise KernelError("gemm_skinny_silu: out must be contiguous bfloat16 [>= m, I] on the GPU")
    if unit is not None:
        call("pyre_gemm_skinny_glu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
             out.data_ptr(), m, two_i, w_gate_up.shape[1], *_gate_shape(unit), _stream())
        return
    call("pyre_gemm_skinny_silu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
         out.data_ptr(), m, two_i, w_gate_up.shape[1], _stream())


@lru_cache(maxsize=4096)
def gemm_mid_supports(m: int, n: int, k: int, ldx: int, ldw: int) -> bool:
    from pyre_amd.hip.lib import lib

    return bool(lib().pyre_gemm_mid_supports(m, n, k, ldx, ldw))


def gemm_mid_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, ksplit: int, wide: bool = False) -> None:
    """out[s] (float32 [ksplit, m, N]) = partial sums over k of x[0:m] @ w.T, 1 <= m <= 256. ``wide``:
    a block takes 128 rows of w instead of 64."""
    _skinny_common(x, w, m)
    n = w.shape[0]
    if out.dtype != torch.float32 or not out.is_contiguous() or out.numel() < ksplit * m * n or not out.is_cuda:
        raise KernelError("gemm_mid: out must be contiguous float32 [ksplit, m, N] on the GPU")
    call("pyre_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), m, n,
         w.shape[1], ksplit, int(wide), _stream())


@lru_cache(maxsize=4096)
def gemm_mid_silu_blocks(m: int, two_i: int) -> int:
    from pyre_amd.hip.lib import lib

    return int(lib().pyre_gemm_mid_silu_blocks(m, two_i))


def gemm_mid_silu_bf16(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, m: int,
                       unit: tuple[float, float, float] | None = None) -> None:
    """out[0:m] (bfloat16 [m, I]) = silu(x @ gate.T) * (x @ up.T) with w_gate_up = [gate; up], 1 <= m <= 256;
    ``unit`` as for :func:`gemm_skinny_silu_bf16`."""
    _skinny_common(x, w_gate_up, m)
    two_i = w_gate_up.shape[0]
    if (out.dtype != torch.bfloat16 or not out.is_contiguous() or not out.is_cuda or out.dim() != 2
            or out.shape[1] * 2 != two_i or out.shape[0] < m):
        raise KernelError("gemm_mid_silu: out must be contiguous bfloat16 [>= m, I] on the GPU")
    if unit is not None:
        call("pyre_gemm_mid_glu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
             out.data_ptr(), m, two_i, w_gate_up.shape[1], *_gate_shape(unit), _stream())
        return
    call("pyre_gemm_mid_silu_bf16", x.data_ptr(), x.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
         out.data_ptr(), m, two_i, w_gate_up.shape[1], _stream())


def read_bandwidth(device: str = "cuda:0", gib: float = 2.0, blocks: int = 4096, repeats: int = 10) -> float:
    """Measured streaming-read bandwidth in GB/s (a buffer larger than every cache)."""
    import time

    n = int(gib * (1 << 30)) // 16 * 16
    buf = torch.empty(n, dtype=torch.uint8, device=device)
    buf.zero_()
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    with torch.cuda.device(buf.device):
        for _ in range(2):
            call("pyre_read_probe", buf.data_ptr(), n, blocks, sink.data_ptr(), _stream())
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(repeats):
            call("pyre_read_probe", buf.data_ptr(), n, blocks, sink.data_ptr(), _stream())
        torch.cuda.synchronize()
    return n * repeats / (time.perf_counter() - t) / 1e9


def add_tanhnorm(resid: torch.Tensor, delta: Partials | None, alpha: torch.Tensor, gain: torch.Tensor,
                 shift: torch.Tensor | None, out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """resid += delta (its partial sums and bias, times its ``scale``; the same for ``delta.more``, if any);
    out = tanh(alpha * resid) * gain + shift: a norm that takes no statistic of the row. ``alpha`` holds one
    number and shares its element type with ``gain`` and ``shift``.

    With ``rows`` only those rows are normed, into ``out[0:len(rows)]``, and ``resid`` is left as it was."""
    _dev(resid, alpha, gain, shift, out, rows)
    hidden = resid.shape[-1]
    if resid.dtype != torch.float32 or resid.dim() != 2:
        raise KernelError("add_tanhnorm: the residual stream is float32 [N, H]")
    n = resid.shape[0] if rows is None else rows.numel()
    if out.shape[-1] != hidden or out.shape[0] < n or gain.numel() != hidden or alpha.numel() != 1 or \
            (shift is not None and shift.numel() != hidden):
        raise KernelError("add_tanhnorm: shapes of out / alpha / gain / shift do not fit the residual")
    if alpha.dtype != gain.dtype or (shift is not None and shift.dtype != gain.dtype):
        raise KernelError("add_tanhnorm: alpha, gain and shift share one element type")
    _contig("resid", resid), _contig("out", out), _contig("gain", gain)
    if shift is not None:
        _contig("shift", shift)
    if rows is not None:
        _i32("rows", rows)
    terms = []
    t = delta
    while t is not None:
        if t.rows < resid.shape[0]:
            raise KernelError("add_tanhnorm: a pending term has fewer rows than the residual")
        if t.post is not None or t.outer is not None:
            raise KernelError("add_tanhnorm: a term that is to be normed before it is added is not taken")
        terms.append((*t._args(hidden), float(t.scale)))
        t = t.more
    if len(terms) > 2:
        raise KernelError("add_tanhnorm: at most two pending terms")
    while len(terms) < 2:
        terms.append((None, 0, 0, 0, None, 0, 1.0))
    call("pyre_add_tanhnorm", resid.data_ptr(), *terms[0], *terms[1], alpha.data_ptr(), gain.data_ptr(), _ptr(shift),
         dtype_code(gain), out.data_ptr(), dtype_code(out), _ptr(rows), n, hidden, _stream())


def softcap_(x: torch.Tensor, cap: float) -> None:
    """x <- cap * tanh(x / cap) in place (contiguous float32)."""
    _dev(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("softcap_: contiguous float32 expected")
    call("pyre_softcap", x.data_ptr(), x.numel(), float(cap), _stream())


def rope_tied_write(proj: Partials, col0: int, q_out: torch.Tensor, k_cache: torch.Tensor | None,
                    v_cache: torch.Tensor | None, cos: torch.Tensor | None, sin: torch.Tensor | None, rot: int,
                    positions: torch.Tensor, slots: torch.Tensor | None, n: int, nq: int, nkv: int, d: int,
                    page_size: int) -> None:
    """Finish a step's input product from column ``col0`` on (``nq`` query heads, then ``nkv`` key heads, of ``d``;
    ``proj.bias`` over these columns): the first ``rot`` elements of every head turned by position (element e with
    e + rot/2, ``cos`` / ``sin`` float32 [positions, rot/2]), queries to ``q_out [N, nq*d]``, the turned keys to
    ``k_cache`` and the keys as projected to ``v_cache`` (both ``[pages, nkv, page, d]``) at ``slots``."""
    _dev(proj.data, proj.bias, q_out, k_cache, v_cache, cos, sin, positions, slots)
    width = (nq + nkv) * d
    if col0 < 0 or col0 + width > proj.width:
        raise KernelError(f"columns {col0}..{col0 + width} lie outside the product's {proj.width}")
    if proj.bias is not None and proj.bias.numel() != width:
        raise KernelError(f"rope_tied_write: the bias has {proj.bias.numel()} entries, {width} expected")
    if proj.rows < n or q_out.numel() < n * nq * d:
        raise KernelError("rope_tied_write: buffers are smaller than the batch")
    _contig("q_out", q_out), _i32("positions", positions, n)
    if rot:
        if cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32 or \
                cos.shape[1] != rot // 2 or tuple(sin.shape) != tuple(cos.shape):
            raise KernelError("rope_tied_write: cos and sin are float32 [positions, rot / 2]")
        _contig("cos", cos), _contig("sin", sin)
    write = k_cache is not None
    cache_dt = dtype_code(q_out)
    if write:
        if v_cache is None or slots is None:
            raise KernelError("rope_tied_write: k cache without v cache or slots")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, d) or tuple(v_cache.shape) != tuple(k_cache.shape) \
                or k_cache.dtype != v_cache.dtype:
            raise KernelError(f"rope_tied_write: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                              f"nkv={nkv} page={page_size} d={d}")
        cache_dt = dtype_code(k_cache)
    call("pyre_rope_tied_write", proj.data.data_ptr(), dtype_code(proj.data), proj.count, proj.stride, proj.width, col0,
         _ptr(proj.bias), dtype_code(proj.bias) if proj.bias is not None else 0, q_out.data_ptr(), dtype_code(q_out),
         _ptr(k_cache), _ptr(v_cache), cache_dt, _ptr(cos) if rot else None, _ptr(sin) if rot else None, int(rot),
         positions.data_ptr(), _ptr(slots), n, nq, nkv, d, page_size, 1 if write else 0, _stream())


def latent_write(proj: Partials, col0: int, q_out: torch.Tensor, c_cache: torch.Tensor | None,
                 gain: torch.Tensor | None, eps: float, slots: torch.Tensor | None, n: int, q_width: int, rank: int,
                 page_size: int) -> None:
    """Finish a step's input product from column ``col0`` on: ``q_width`` columns of queries to ``q_out [N, q_width]``
    and, if ``c_cache [pages, 1, page, rank]`` is given, the ``rank`` columns behind them divided by their root mean
    square (``eps`` inside the root), times ``gain``, to the cache at ``slots``."""
    _dev(proj.data, q_out, c_cache, gain, slots)
    write = c_cache is not None
    args = _proj_args(proj, col0, q_width + (rank if write else 0))
    if proj.rows < n or q_out.numel() < n * q_width:
        raise KernelError("latent_write: buffers are smaller than the batch")
    _contig("q_out", q_out)
    cache_dt = dtype_code(q_out)
    if write:
        if gain is None or slots is None or gain.numel() != rank:
            raise KernelError("latent_write: a cache write needs a gain over the rank and slots")
        _i32("slots", slots, n), _contig("c_cache", c_cache), _contig("gain", gain)
        if tuple(c_cache.shape[1:]) != (1, page_size, rank):
            raise KernelError(f"latent_write: cache {tuple(c_cache.shape)} does not fit page={page_size} rank={rank}")
        cache_dt = dtype_code(c_cache)
    call("pyre_latent_write", *args, q_out.data_ptr(), dtype_code(q_out), _ptr(c_cache), cache_dt, _ptr(gain),
         dtype_code(gain) if gain is not None else 0, float(eps), _ptr(slots), n, q_width, rank, page_size,
         1 if write else 0, _stream())


HEAD_MATMUL_MAX_IN = 768  #: the widest head that the per-head product takes (latent.hip)


def head_matmul(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, n: int) -> None:
    """out[n, h, :] = x[n, h, :] @ w[h] for every head: ``w [heads, din, dout]``, ``x [>= n, heads * din]`` and
    ``out [>= n, heads * dout]`` with contiguous rows, one element type."""
    _dev(x, w, out)
    if w.dim() != 3 or not w.is_contiguous():
        raise KernelError("head_matmul: w is contiguous [heads, din, dout]")
    heads, din, dout = w.shape
    if not (x.dtype == w.dtype == out.dtype):
        raise KernelError("head_matmul: one element type for x, w and out")
    if x.dim() != 2 or out.dim() != 2 or x.stride(1) != 1 or out.stride(1) != 1 or x.shape[1] < heads * din or \
            out.shape[1] < heads * dout or x.shape[0] < n or out.shape[0] < n:
        raise KernelError("head_matmul: x [>= n, heads*din] and out [>= n, heads*dout] with contiguous rows expected")
    if din > HEAD_MATMUL_MAX_IN:
        raise KernelError(f"head_matmul: heads of {din} elements are more than {HEAD_MATMUL_MAX_IN}")
    call("pyre_head_matmul", x.data_ptr(), x.stride(0), w.data_ptr(), out.data_ptr(), out.stride(0), dtype_code(x), n,
         heads, din, dout, _stream())


ROUTE_MAX_EXPERTS = 512  #: the most experts that the routing kernel chooses among (moe.hip)


def route_topk(z: Partials, gates: torch.Tensor, n: int, top: int, softmax: bool = False, extra: int = 0) -> None:
    """gates[n, e] (float32 [N, experts + extra]) = s_e / (sum of the chosen s + 1e-20) for the ``top`` experts of largest
    s = sigmoid(z) (the lower index among equals), 0 for the others; ``z`` the router product's partial sums.
    ``softmax``: the chosen experts' weights are the softmax over their logits alone. The last ``extra`` columns of the
    product are no experts but gates of their own, whose sigmoid is written behind the experts' weights."""
    _dev(z.data, z.bias, gates)
    experts = z.width - int(extra)
    if gates.dtype != torch.float32 or not gates.is_contiguous() or gates.dim() != 2 or gates.shape[1] != z.width or \
            gates.shape[0] < n or z.rows < n:
        raise KernelError("route_topk: gates are contiguous float32 [>= n, experts + extra]")
    if extra < 0 or not (0 < top <= experts <= ROUTE_MAX_EXPERTS):
        raise KernelError(f"route_topk: {top} of {experts} experts is not a choice this kernel makes")
    call("pyre_route_topk", *z._args(z.width), gates.data_ptr(), n, experts, int(top), int(bool(softmax)), int(extra),
         _stream())


def expert_act(up: Partials, gates: torch.Tensor, out: torch.Tensor, n: int, experts: int, ff: int, shared_ff: int) -> None:
    """out[n, e*ff + j] = gates[n, e] * relu(up[n, e*ff + j])^2 for the routed experts, relu(up)^2 for the
    ``shared_ff`` columns behind them; ``up`` the partial sums of the product over all experts' matrices."""
    _dev(up.data, gates, out)
    width = experts * ff + shared_ff
    if up.bias is not None:
        raise KernelError("expert_act: a pending bias is not supported")
    if up.width != width or up.rows < n or out.shape[-1] != width or out.shape[0] < n:
        raise KernelError("expert_act: the product's width does not fit experts * ff + shared_ff")
    if gates.dtype != torch.float32 or not gates.is_contiguous() or gates.shape[-1] != experts or gates.shape[0] < n:
        raise KernelError("expert_act: gates are contiguous float32 [>= n, experts]")
    _contig("out", out)
    call("pyre_expert_act", up.data.data_ptr(), dtype_code(up.data), up.count, up.stride, gates.data_ptr(),
         out.data_ptr(), dtype_code(out), n, experts, ff, shared_ff, _stream())


def _term_args(t: Partials | None, hidden: int, what: str):
    """(data, dtype, count, stride, own gain, its dtype, factor) of one pending term of :func:`add_rms_terms`."""
    if t is None:
        return (None, 0, 0, 0, None, 0, 1.0), None
    if t.bias is not None:
        raise KernelError(f"{what}: a pending bias is not taken")
    if t.width != hidden:
        raise KernelError(f"{what}: a pending term is {t.width} wide, {hidden} expected")
    gain = None
    if t.post is not None:
        if t.post.kind != "rms" or t.post.scale is not None:
            raise KernelError(f"{what}: a term's own norm must be an RMS norm without a layer scale")
        gain = t.post.gain
        _dev(gain), _contig("post.gain", gain)
        if gain.numel() != hidden:
            raise KernelError(f"{what}: a term's gain does not fit the residual")
    return (t.data.data_ptr(), dtype_code(t.data), t.count, t.stride, _ptr(gain),
            dtype_code(gain) if gain is not None else 0, float(t.scale)), t.post


def add_rms_terms(resid: torch.Tensor, delta: Partials | None, gain: torch.Tensor | None, eps: float,
                  out: torch.Tensor | None, rows: torch.Tensor | None = None) -> None:
    """resid += y; out = gain is None ? resid : resid / sqrt(mean(resid^2) + eps) * gain, rounded to ``out``'s type.

    y is the pending term: up to two terms (``delta`` and ``delta.more``), each the sum of its partial sums, divided by
    its root mean square and times its gain if it carries a norm of its own (``post``, kind "rms"), times its factor
    (``scale``); their sum goes through ``delta.outer`` (an RMS norm again) if that is given. With ``rows`` only those
    rows are handled, into ``out[0:len(rows)]``, and ``resid`` is left as it was."""
    _dev(resid, gain, out, rows)
    hidden = resid.shape[-1]
    if resid.dtype != torch.float32 or resid.dim() != 2:
        raise KernelError("add_rms_terms: the residual stream is float32 [N, H]")
    _contig("resid", resid)
    n = resid.shape[0] if rows is None else rows.numel()
    if out is not None:
        if out.shape[-1] != hidden or out.shape[0] < n:
            raise KernelError("add_rms_terms: out does not fit the residual")
        _contig("out", out)
    if gain is not None:
        if out is None or gain.numel() != hidden:
            raise KernelError("add_rms_terms: the output norm's gain does not fit the residual")
        _contig("gain", gain)
    if rows is not None:
        _i32("rows", rows)
    more = delta.more if delta is not None else None
    if more is not None and (more.more is not None or more.outer is not None):
        raise KernelError("add_rms_terms: at most two pending terms, the norm of their sum on the first")
    for t in (delta, more):
        if t is not None and t.rows < resid.shape[0]:
            raise KernelError("add_rms_terms: a pending term has fewer rows than the residual")
    a, post_a = _term_args(delta, hidden, "add_rms_terms")
    b, post_b = _term_args(more, hidden, "add_rms_terms")
    inner = [p.eps for p in (post_a, post_b) if p is not None]
    if len(set(inner)) > 1:
        raise KernelError("add_rms_terms: the terms' own norms share one eps")
    outer = delta.outer if delta is not None else None
    o = (None, 0, 0.0)
    if outer is not None:
        if outer.kind != "rms" or outer.scale is not None or outer.gain.numel() != hidden:
            raise KernelError("add_rms_terms: the norm of the sum is an RMS norm with a gain over the hidden size")
        _dev(outer.gain), _contig("outer.gain", outer.gain)
        o = (outer.gain.data_ptr(), dtype_code(outer.gain), float(outer.eps))
    call("pyre_add_rms_terms", resid.data_ptr(), *a, *b, float(inner[0]) if inner else 0.0, *o, _ptr(gain),
         dtype_code(gain) if gain is not None else 0, float(eps), _ptr(out), dtype_code(out) if out is not None else 0,
         _ptr(rows), n, hidden, _stream())


def bigram_embed(table: torch.Tensor, pairs: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
                 seq_of_token: torch.Tensor, q_start: torch.Tensor, state: torch.Tensor, state_slots: torch.Tensor,
                 out: torch.Tensor, buckets: int, mul_prev: int, mul_cur: int) -> None:
    """out[n] = float32(table[ids[n]]) + float32(pairs[row]), row = (previous token * mul_prev + ids[n] * mul_cur) mod
    buckets, or ``buckets`` at position 0. The previous token of a request's first token of the step is
    ``state[slot, 0]`` (float32, an integer value), which then takes the request's last token of the step."""
    _dev(table, pairs, ids, positions, seq_of_token, q_start, state, state_slots, out)
    n, hidden = out.shape
    if table.dim() != 2 or table.shape[1] != hidden or out.dtype != torch.float32 or table.dtype != pairs.dtype:
        raise KernelError("bigram_embed: tables [V, H] / [buckets + 1, H] of one type and float32 out [N, H] expected")
    if tuple(pairs.shape) != (buckets + 1, hidden) or buckets <= 0 or mul_prev < 0 or mul_cur < 0:
        raise KernelError(f"bigram_embed: the pair table is [{buckets + 1}, {hidden}]")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 2 or state.shape[1] != 1:
        raise KernelError("bigram_embed: the state is contiguous float32 [slots, 1]")
    _contig("table", table), _contig("pairs", pairs), _contig("out", out)
    _i32("ids", ids, n), _i32("positions", positions, n), _i32("seq_of_token", seq_of_token, n)
    _i32("q_start", q_start), _i32("state_slots", state_slots)
    call("pyre_bigram_embed", table.data_ptr(), pairs.data_ptr(), dtype_code(table), ids.data_ptr(), positions.data_ptr(),
         seq_of_token.data_ptr(), q_start.data_ptr(), state.data_ptr(), state_slots.data_ptr(), out.data_ptr(), n, hidden,
         int(buckets), int(mul_prev), int(mul_cur), _stream())


CONV_MAX_TAPS = 16  #: the most taps of the short convolution (conv_attention.hip)


def conv_qkv_write(proj: Partials, col0: int, taps_w: torch.Tensor | None, conv_state: torch.Tensor | None,
                   state_slots: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, n_seqs: int,
                   q_gain: torch.Tensor | None, k_gain: torch.Tensor | None, eps: float, cos: torch.Tensor | None,
                   sin: torch.Tensor | None, rot: int, neighbours: bool, positions: torch.Tensor, q_out: torch.Tensor,
                   k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, gate_out: torch.Tensor | None,
                   slots: torch.Tensor | None, n: int, nq: int, nkv: int, dk: int, dv: int, page_size: int) -> None:
    """Finish a step's input product from column ``col0`` on (``nq`` query and ``nkv`` key heads of ``dk``, ``nkv`` value
    heads of ``dv``, then ``nq * dv`` gate columns if ``gate_out`` is given). Queries, keys and values first go through a
    causal convolution over the request's tokens, ``taps_w`` float32 [taps, channels] (None: none), whose inputs before
    the step's first token come from ``conv_state`` (float32 [slots, taps - 1, channels], the request's last projected
    rows; it is brought up to date after every token has read it). Then queries and keys are divided by their root mean
    square per head, times ``q_gain`` / ``k_gain`` over ``dk`` (None: not normed), and their first ``rot`` elements turned
    by position (``neighbours``: element 2e with 2e + 1, else e with e + rot/2). Queries go to ``q_out [N, nq*dk]``, keys and
    values to their pages at ``slots``, sigmoid(gate) to float32 ``gate_out [N, nq*dv]``."""
    _dev(proj.data, taps_w, conv_state, state_slots, seq_of_token, q_start, q_gain, k_gain, cos, sin, positions, q_out,
         k_cache, v_cache, gate_out, slots)
    channels = (nq + nkv) * dk + nkv * dv
    args = _proj_args(proj, col0, channels + (nq * dv if gate_out is not None else 0))
    if proj.rows < n or q_out.numel() < n * nq * dk:
        raise KernelError("conv_qkv_write: buffers are smaller than the batch")
    _contig("q_out", q_out), _i32("positions", positions, n), _i32("seq_of_token", seq_of_token, n)
    _i32("q_start", q_start, n_seqs + 1), _i32("state_slots", state_slots, n_seqs)
    taps = 0
    if taps_w is not None:
        taps = taps_w.shape[0]
        if taps_w.dtype != torch.float32 or not taps_w.is_contiguous() or tuple(taps_w.shape) != (taps, channels) or \
                not (1 <= taps <= CONV_MAX_TAPS):
            raise KernelError(f"conv_qkv_write: the taps are contiguous float32 [1..{CONV_MAX_TAPS}, {channels}]")
        if taps > 1:
            if conv_state is None or conv_state.dtype != torch.float32 or not conv_state.is_contiguous() or \
                    tuple(conv_state.shape[1:]) != (taps - 1, channels):
                raise KernelError(f"conv_qkv_write: the state is contiguous float32 [slots, {taps - 1}, {channels}]")
    for name, g in (("q_gain", q_gain), ("k_gain", k_gain)):
        if g is not None and (g.dtype != torch.float32 or g.numel() != dk or not g.is_contiguous()):
            raise KernelError(f"conv_qkv_write: {name} is contiguous float32 [{dk}]")
    if (q_gain is None) != (k_gain is None):
        raise KernelError("conv_qkv_write: queries and keys are normed together or not at all")
    if rot:
        if rot % 2 or rot > dk or cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
                or cos.dim() != 2 or cos.shape[1] != rot // 2 or tuple(cos.shape) != tuple(sin.shape):
            raise KernelError("conv_qkv_write: cos and sin are float32 [positions, rot / 2], rot even and within the head")
        _contig("cos", cos), _contig("sin", sin)
    write = k_cache is not None
    cache_dt = dtype_code(q_out)
    if write:
        if v_cache is None or slots is None:
            raise KernelError("conv_qkv_write: k cache without v cache or slots")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, dk) or tuple(v_cache.shape[1:]) != (nkv, page_size, dv) \
                or k_cache.dtype != v_cache.dtype:
            raise KernelError(f"conv_qkv_write: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                              f"nkv={nkv} page={page_size} dk={dk} dv={dv}")
        cache_dt = dtype_code(k_cache)
    if gate_out is not None and (gate_out.dtype != torch.float32 or gate_out.numel() < n * nq * dv or not gate_out.is_contiguous()):
        raise KernelError("conv_qkv_write: gates are contiguous float32 [N, nq*dv]")
    call("pyre_conv_qkv_write", *args, _ptr(taps_w), taps, _ptr(conv_state) if taps > 1 else None, state_slots.data_ptr(),
         seq_of_token.data_ptr(), q_start.data_ptr(), n_seqs, _ptr(q_gain), _ptr(k_gain), float(eps),
         _ptr(cos) if rot else None, _ptr(sin) if rot else None, int(rot), int(bool(neighbours)), positions.data_ptr(),
         q_out.data_ptr(), dtype_code(q_out), _ptr(k_cache), _ptr(v_cache), cache_dt, _ptr(gate_out), _ptr(slots), n, nq,
         nkv, dk, dv, page_size, 1 if write else 0, _stream())


def retention_prepare(proj: Partials, col0: int, log_decay: torch.Tensor, cos: torch.Tensor | None,
                      sin: torch.Tensor | None, rot: int, neighbours: bool, positions: torch.Tensor, kscale: float,
                      x: torch.Tensor, n: int, heads: int, dk: int, dv: int) -> None:
    """Finish the input product from column ``col0`` on (q, k: heads*dk each; v, g: heads*dv each) into the float32 rows
    [q | k | log decay | v | g] that the recurrent kernels share: the first ``rot`` elements of every query and key head
    turned by position, the keys then times ``kscale``; every key channel of head h gets ``log_decay[h]``."""
    _dev(proj.data, log_decay, cos, sin, positions, x)
    args = _proj_args(proj, col0, 2 * heads * dk + 2 * heads * dv)
    if log_decay.dtype != torch.float32 or log_decay.numel() != heads or not log_decay.is_contiguous():
        raise KernelError("retention_prepare: one float32 logarithm of a decay per head")
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[-1] != gla_row_width(heads, dk, dv) or x.shape[0] < n \
            or proj.rows < n:
        raise KernelError("retention_prepare: x is contiguous float32 [>= n, 3*heads*dk + 2*heads*dv]")
    _i32("positions", positions, n)
    if rot:
        if rot % 2 or rot > dk or cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
                or cos.dim() != 2 or cos.shape[1] != rot // 2 or tuple(cos.shape) != tuple(sin.shape):
            raise KernelError("retention_prepare: cos and sin are float32 [positions, rot / 2], rot even and within the head")
        _contig("cos", cos), _contig("sin", sin)
    call("pyre_retention_prepare", *args, log_decay.data_ptr(), _ptr(cos) if rot else None, _ptr(sin) if rot else None,
         int(rot), int(bool(neighbours)), positions.data_ptr(), float(kscale), x.data_ptr(), n, heads, dk, dv, _stream())


def route_grouped(z: Partials, correction: torch.Tensor | None, gates: torch.Tensor, n: int, top: int, groups: int,
                  keep_groups: int) -> None:
    """gates[n, e] (float32 [N, experts]) = s_e for the ``top`` experts of largest s_e + correction_e among the experts
    of the ``keep_groups`` of ``groups`` equal groups of neighbours whose largest such number is largest (the lower index
    among equals, of groups as of experts), 0 for the others; s = softmax(z) over all experts, ``z`` the router product's
    partial sums."""
    _dev(z.data, z.bias, correction, gates)
    experts = z.width
    if gates.dtype != torch.float32 or not gates.is_contiguous() or gates.dim() != 2 or gates.shape[1] != experts or \
            gates.shape[0] < n or z.rows < n:
        raise KernelError("route_grouped: gates are contiguous float32 [>= n, experts]")
    if not (0 < experts <= ROUTE_MAX_EXPERTS) or groups <= 0 or experts % groups or not (0 < keep_groups <= groups) or \
            not (0 < top <= keep_groups * (experts // groups)):
        raise KernelError(f"route_grouped: {top} of {experts} experts in {keep_groups} of {groups} groups is not a choice "
                          "this kernel makes")
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != experts or
                                   not correction.is_contiguous()):
        raise KernelError("route_grouped: the correction is contiguous float32 [experts]")
    call("pyre_route_grouped", *z._args(experts), _ptr(correction), gates.data_ptr(), n, experts, int(top), int(groups),
         int(keep_groups), _stream())


def expert_glu_act(gu: Partials, gates: torch.Tensor, out: torch.Tensor, n: int, experts: int, ff: int,
                   shared_ff: int = 0, shared_gate: int = -1) -> None:
    """out[n, e*ff + j] = gates[n, e] * silu(g) * u with g = gu[n, e*ff + j] and u = gu[n, width + e*ff + j]: the
    experts' gated units, weighted (``gates [N, >= experts]`` with contiguous rows; columns of an expert that the token
    does not take are not read and written as zero). ``shared_ff`` columns behind the routed experts' (width = experts*ff
    + shared_ff) are a shared expert's, weighted by ``gates[n, shared_gate]`` (``shared_gate`` < 0: by one)."""
    _dev(gu.data, gates, out)
    width = experts * ff + shared_ff
    if shared_ff < 0 or shared_gate >= gates.shape[1]:
        raise KernelError("expert_glu_act: the shared expert's gate lies outside the rows of weights")
    if gu.bias is not None:
        raise KernelError("expert_glu_act: a pending bias is not supported")
    if gu.width != 2 * width or gu.rows < n or out.shape[-1] != width or out.shape[0] < n:
        raise KernelError("expert_glu_act: the product's width does not fit 2 * (experts * ff + shared_ff)")
    if gates.dtype != torch.float32 or gates.dim() != 2 or gates.stride(1) != 1 or gates.shape[1] < experts or gates.shape[0] < n:
        raise KernelError("expert_glu_act: gates are float32 [>= n, >= experts] with contiguous rows")
    _contig("out", out)
    call("pyre_expert_glu_act", gu.data.data_ptr(), dtype_code(gu.data), gu.count, gu.stride, gates.data_ptr(),
         gates.stride(0), out.data_ptr(), dtype_code(out), n, experts, ff, int(shared_ff), int(shared_gate), _stream())


def add_weighted_rows(p: Partials, h: torch.Tensor, gates: torch.Tensor, first: int, count: int, n: int) -> None:
    """p[0][n, :] += (gates[n, first] + ... + gates[n, first + count - 1]) * h[n, :]: experts that hand their input back,
    added to the first partial sum (float32) of the experts' product."""
    _dev(p.data, h, gates)
    if p.data.dtype != torch.float32 or p.bias is not None:
        raise KernelError("add_weighted_rows: float32 partial sums without a bias expected")
    if h.dim() != 2 or h.shape[1] != p.width or h.stride(1) != 1 or h.shape[0] < n or p.rows < n:
        raise KernelError("add_weighted_rows: h [>= n, width] with contiguous rows expected")
    if gates.dtype != torch.float32 or gates.dim() != 2 or gates.stride(1) != 1 or first < 0 or count <= 0 or \
            first + count > gates.shape[1] or gates.shape[0] < n:
        raise KernelError("add_weighted_rows: gates are float32 [>= n, >= first + count] with contiguous rows")
    call("pyre_add_weighted_rows", p.data.data_ptr(), h.data_ptr(), dtype_code(h), h.stride(0), gates.data_ptr(),
         gates.stride(0), int(first), int(count), n, p.width, _stream())


def relu2(up: Partials, out: torch.Tensor, n: int) -> None:
    """out[n, j] = max(up[n, j], 0)^2, the partial sums added first."""
    _dev(up.data, out)
    if up.bias is not None:
        raise KernelError("relu2: a pending bias is not supported")
    if up.rows < n or out.shape[-1] != up.width or out.shape[0] < n:
        raise KernelError("relu2: the output does not fit the product")
    _contig("out", out)
    call("pyre_expert_act", up.data.data_ptr(), dtype_code(up.data), up.count, up.stride, None,
         out.data_ptr(), dtype_code(out), n, 0, 4, up.width, _stream())


def _proj_bias_args(proj: Partials, col0: int, width: int):
    """As :func:`_proj_args` for the kernels that add the product's pending bias themselves: float32 over all its columns."""
    if col0 < 0 or col0 + width > proj.width:
        raise KernelError(f"columns {col0}..{col0 + width} lie outside the product's {proj.width}")
    bias = proj.bias
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != proj.width or not bias.is_contiguous()):
        raise KernelError(f"a fused input product's bias is contiguous float32 [{proj.width}]")
    _dev(proj.data, bias)
    return (proj.data.data_ptr(), dtype_code(proj.data), proj.count, proj.stride, proj.width, col0, _ptr(bias))


def _rot_tables(what: str, cos, sin, rot: int, dk: int):
    if not rot:
        return None, None
    if rot % 2 or rot > dk or cos is None or sin is None or cos.dtype != torch.float32 or sin.dtype != torch.float32 \
            or cos.dim() != 2 or cos.shape[1] != rot // 2 or tuple(cos.shape) != tuple(sin.shape):
        raise KernelError(f"{what}: cos and sin are float32 [positions, rot / 2], rot even and within the head")
    _contig("cos", cos), _contig("sin", sin)
    return cos.data_ptr(), sin.data_ptr()


def wide_norm_qkv_write(proj: Partials, col0: int, q_gain: torch.Tensor | None, k_gain: torch.Tensor | None, eps: float,
                        cos: torch.Tensor | None, sin: torch.Tensor | None, rot: int, positions: torch.Tensor,
                        q_out: torch.Tensor, k_cache: torch.Tensor | None, v_cache: torch.Tensor | None,
                        slots: torch.Tensor | None, n: int, nq: int, nkv: int, dk: int, dv: int, page_size: int) -> None:
    """Finish a step's input product from column ``col0`` on (``nq`` query heads of ``dk``, then ``nkv`` key heads of ``dk``
    and ``nkv`` value heads of ``dv``; ``nkv`` = 0: queries alone), its pending bias included. Queries are divided by their
    root mean square over all ``nq * dk`` columns at once, times ``q_gain`` over those columns (None: not normed), keys
    likewise over their ``nkv * dk`` with ``k_gain``; then the first ``rot`` elements of every head are turned by position,
    element e with e + rot/2. Queries go to ``q_out [N, nq*dk]``, keys and values to their pages at ``slots``
    (``k_cache`` None: nothing is stored)."""
    _dev(q_gain, k_gain, cos, sin, positions, q_out, k_cache, v_cache, slots)
    args = _proj_bias_args(proj, col0, (nq + nkv) * dk + nkv * dv)
    if proj.rows < n or q_out.numel() < n * nq * dk:
        raise KernelError("wide_norm_qkv_write: buffers are smaller than the batch")
    _contig("q_out", q_out), _i32("positions", positions, n)
    for name, g, width in (("q_gain", q_gain, nq * dk), ("k_gain", k_gain, nkv * dk)):
        if g is not None and (g.dtype != torch.float32 or g.numel() != width or not g.is_contiguous()):
            raise KernelError(f"wide_norm_qkv_write: {name} is contiguous float32 [{width}]")
    c, s = _rot_tables("wide_norm_qkv_write", cos, sin, rot, dk)
    write = k_cache is not None
    cache_dt = dtype_code(q_out)
    if write:
        if v_cache is None or slots is None or nkv <= 0:
            raise KernelError("wide_norm_qkv_write: k cache without v cache, slots or key heads")
        _i32("slots", slots, n), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        if tuple(k_cache.shape[1:]) != (nkv, page_size, dk) or tuple(v_cache.shape[1:]) != (nkv, page_size, dv) \
                or k_cache.dtype != v_cache.dtype:
            raise KernelError(f"wide_norm_qkv_write: caches {tuple(k_cache.shape)} / {tuple(v_cache.shape)} do not fit "
                              f"nkv={nkv} page={page_size} dk={dk} dv={dv}")
        cache_dt = dtype_code(k_cache)
    call("pyre_wide_norm_qkv_write", *args, _ptr(q_gain), _ptr(k_gain), float(eps), c, s, int(rot), positions.data_ptr(),
         q_out.data_ptr(), dtype_code(q_out), _ptr(k_cache), _ptr(v_cache), cache_dt, _ptr(slots), n, nq, nkv, dk, dv,
         page_size, 1 if write else 0, _stream())


GDR_MAX_HEAD = 256   #: the largest key or value head of the gated delta rule's kernels (delta_rule.hip)
GDR_MAX_RANK = 512   #: the widest low-rank input of its decay and of its gate


def gdr_row_width(heads: int, kv_heads: int, dk: int, dv: int) -> int:
    """Columns of the float32 rows [q | k | decay | v | gate | beta] that the gated delta rule's kernels share (rounded up
    to a multiple of four, so that every row starts on 16 bytes)."""
    return (2 * kv_heads * dk + heads * dk + 2 * heads * dv + heads + 3) // 4 * 4


def gdr_prepare(proj: Partials, col0: int, taps_w: torch.Tensor | None, conv_state: torch.Tensor | None,
                state_slots: torch.Tensor, seq_of_token: torch.Tensor, q_start: torch.Tensor, n_seqs: int,
                a2: torch.Tensor, dt_bias: torch.Tensor, rate: torch.Tensor, g2: torch.Tensor, unit_eps: float,
                x: torch.Tensor, n: int, heads: int, kv_heads: int, dk: int, dv: int) -> None:
    """Finish the input product from column ``col0`` on (q, k: kv_heads*dk each; v: heads*dv; beta: heads; then the low-rank
    inputs of the decay and of the gate) into the float32 rows ``x``: q, k, v through the short causal convolution
    (``taps_w`` float32 [taps, channels], inputs before the step from ``conv_state [slots, taps - 1, channels]``, which is
    brought up to date afterwards) and SiLU; q and k unit vectors per head (``unit_eps`` beside the sum of squares), q times
    dk^-1/2; beta = sigmoid; decay = exp(rate[h] * softplus(a2 @ low + dt_bias)); gate = sigmoid(g2 @ low')."""
    _dev(taps_w, conv_state, state_slots, seq_of_token, q_start, a2, dt_bias, rate, g2, x)
    rank_a, rank_g = a2.shape[1], g2.shape[1]
    channels = 2 * kv_heads * dk + heads * dv
    args = _proj_bias_args(proj, col0, channels + heads + rank_a + rank_g)
    if tuple(a2.shape) != (heads * dk, rank_a) or tuple(g2.shape) != (heads * dv, rank_g):
        raise KernelError("gdr_prepare: the second matrices are [heads*dk, rank] and [heads*dv, rank']")
    _contig("a2", a2), _contig("g2", g2)
    for name, t, size in (("dt_bias", dt_bias, heads * dk), ("rate", rate, heads)):
        if t.dtype != torch.float32 or t.numel() != size or not t.is_contiguous():
            raise KernelError(f"gdr_prepare: {name} is contiguous float32 [{size}]")
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[-1] != gdr_row_width(heads, kv_heads, dk, dv) or \
            x.shape[0] < n or proj.rows < n:
        raise KernelError("gdr_prepare: x is contiguous float32 [>= n, gdr_row_width(...)]")
    _i32("seq_of_token", seq_of_token, n), _i32("q_start", q_start, n_seqs + 1), _i32("state_slots", state_slots, n_seqs)
    taps = 0
    if taps_w is not None:
        taps = taps_w.shape[0]
        if taps_w.dtype != torch.float32 or not taps_w.is_contiguous() or tuple(taps_w.shape) != (taps, channels) or \
                not (1 <= taps <= CONV_MAX_TAPS):
            raise KernelError(f"gdr_prepare: the taps are contiguous float32 [1..{CONV_MAX_TAPS}, {channels}]")
        if taps > 1 and (conv_state is None or conv_state.dtype != torch.float32 or not conv_state.is_contiguous() or
                         tuple(conv_state.shape[1:]) != (taps - 1, channels)):
            raise KernelError(f"gdr_prepare: the state is contiguous float32 [slots, {taps - 1}, {channels}]")
    call("pyre_gdr_prepare", *args, _ptr(taps_w), taps, _ptr(conv_state) if taps > 1 else None, state_slots.data_ptr(),
         seq_of_token.data_ptr(), q_start.data_ptr(), n_seqs, a2.data_ptr(), dtype_code(a2), dt_bias.data_ptr(),
         rate.data_ptr(), g2.data_ptr(), dtype_code(g2), float(unit_eps), x.data_ptr(), n, heads, kv_heads, dk, dv,
         rank_a, rank_g, _stream())


def gdr_scan(x: torch.Tensor, state: torch.Tensor, o: torch.Tensor, q_start: torch.Tensor, state_slots: torch.Tensor,
             n_seqs: int, heads: int, kv_heads: int, dk: int, dv: int, max_tokens: int = 0) -> None:
    """The gated delta rule over each request's tokens of the step, from and into ``state [slots, heads, dv, dk]`` (the
    state S [dk, dv] of a head kept column by column): S <- diag(decay) S; u = beta (v - S^T k); S <- S + k u^T; ``o``
    (float32 [N, heads*dv]) receives S^T q. ``max_tokens``: the most tokens that one request brings (0: unknown); a step
    of single tokens is launched with less shared memory a block."""
    _dev(x, state, o, q_start, state_slots)
    for name, t in (("x", x), ("state", state), ("o", o)):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError(f"gdr_scan: {name} is contiguous float32")
    if tuple(state.shape[1:]) != (heads, dv, dk) or x.shape[-1] != gdr_row_width(heads, kv_heads, dk, dv) or \
            o.shape[-1] != heads * dv:
        raise KernelError("gdr_scan: shapes do not fit the head geometry")
    _i32("q_start", q_start, n_seqs + 1), _i32("state_slots", state_slots, n_seqs)
    call("pyre_gdr_scan", x.data_ptr(), state.data_ptr(), o.data_ptr(), q_start.data_ptr(), state_slots.data_ptr(), n_seqs,
         int(max_tokens), heads, kv_heads, dk, dv, _stream())


def gdr_finish(o: torch.Tensor, x: torch.Tensor, gain: torch.Tensor, eps: float, out_scale: float, out: torch.Tensor,
               n: int, heads: int, kv_heads: int, dk: int, dv: int) -> None:
    """out[n, h*dv + e] = o / rms(o over dv) * gain[e] * gate * out_scale, the gate from the rows ``x``; ``out`` has
    contiguous rows."""
    _dev(o, x, gain, out)
    if o.dtype != torch.float32 or x.dtype != torch.float32 or not o.is_contiguous() or not x.is_contiguous():
        raise KernelError("gdr_finish: o and x are contiguous float32")
    if gain.numel() != dv or out.dim() != 2 or out.stride(1) != 1 or out.shape[1] < heads * dv or out.shape[0] < n or \
            x.shape[-1] != gdr_row_width(heads, kv_heads, dk, dv) or o.shape[-1] != heads * dv:
        raise KernelError("gdr_finish: gain [dv] and out [>= n, >= heads*dv] expected")
    _contig("gain", gain)
    call("pyre_gdr_finish", o.data_ptr(), x.data_ptr(), gain.data_ptr(), dtype_code(gain), float(eps), float(out_scale),
         out.data_ptr(), dtype_code(out), out.stride(0), n, heads, kv_heads, dk, dv, _stream())


def token_side_gate(z: Partials, table: torch.Tensor, first: int, ids: torch.Tensor, out: torch.Tensor, n: int) -> None:
    """out[n, j] = gelu_tanh(z[n, j]) * table[ids[n], first + j] for the ``z.width`` columns of the narrow product ``z``."""
    _dev(z.data, z.bias, table, ids, out)
    dim = z.width
    if table.dim() != 2 or not table.is_contiguous() or first < 0 or first + dim > table.shape[1]:
        raise KernelError(f"token_side_gate: columns {first}..{first + dim} lie outside the table's {tuple(table.shape)}")
    if out.shape[-1] != dim or out.shape[0] < n or z.rows < n:
        raise KernelError("token_side_gate: the output does not fit the product")
    _contig("out", out), _i32("ids", ids, n)
    call("pyre_token_side_gate", *z._args(dim), table.data_ptr(), dtype_code(table), table.shape[1], int(first),
         ids.data_ptr(), out.data_ptr(), dtype_code(out), n, dim, _stream())
