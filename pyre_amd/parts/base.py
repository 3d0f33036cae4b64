"""What a model is made of: the kinds of parts, what each must provide, and the
table that maps a part's description to the class that runs it.

A model is described by data (:class:`ModelSpec`): an embedding, a list of layer
descriptions (each naming its mixer, feed-forward, norms and their arrangement),
the order in which layers run, a final norm and an output head. Each description
is a small dataclass with a ``kind``; ``register_part(role, kind, cls)`` says which
class runs it. No part knows which model it is in: it sees its own description,
its own tensors and the step's :class:`~pyre_amd.engine.context.StepContext`.

Interfaces (duck-typed; the base classes document them):

``Part``          ``tensor_specs()`` names the checkpoint tensors it needs;
                  ``bind(tensors, runtime)`` takes them (already on the device).
``Mixer``         ``cache_spec()`` says what it keeps per token (tensors in pages, in a
                  layout of its own choice, all tokens or a window) or per request
                  (fixed-size state), or nothing; ``step_arrays()`` names the work
                  lists its kernels want of every step; ``forward(ctx, h, cache) -> Partials`` turns the normed
                  hidden rows into the term to be added to the residual stream.
``FeedForward``   ``forward(ctx, h) -> Partials``.
``Norm``          ``forward(ctx, resid, delta, out, rows=None)``: adds ``delta`` to the
                  fp32 residual stream and writes the normed rows to ``out``.
``PositionEncoding``  ``rotary(runtime) -> (cos, sin, rotary_dim)`` tables indexed by
                  absolute position for mixers that rotate queries and keys, or
                  ``rotary_dim = 0`` for none.
``Block``         ``forward(ctx, state, caches)`` arranges the four above around the
                  residual stream; ``cache_specs()`` lists what the block keeps (one
                  description per cache: a block with one mixer has its mixer's, a block
                  with two has two, in the order in which ``forward`` receives their
                  views) and ``step_arrays()`` what its parts want of every step. The
                  model asks the block, never the parts inside it.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar

# --------------------------------------------------------------------------- tensors


@dataclass(frozen=True)
class TensorSpec:
    """One checkpoint tensor a part needs.

    ``init`` tells the random-weights mode how to draw it: ``"normal"`` (matrices,
    embeddings, biases: N(0, std)), ``"gain"`` (norm gains: 1 + N(0, gain_std)),
    ``"zeros"``, ``"int"`` (integer tables: zeros).
    ``alias_of`` names a tensor that stands in when this one is absent from the
    file (a tied output head). ``init`` may also be ``"normal:<std>"`` for a matrix drawn
    with a deviation of its own.
    """

    name: str
    shape: tuple[int | None, ...]
    init: str = "normal"
    alias_of: str | None = None
    #: a size that only the file knows is None in ``shape`` (the part reads it off the tensor when it
    #: binds); the random-weights mode then draws this shape
    random_shape: tuple[int, ...] | None = None
    #: a tensor that a file may hold though nothing reads it (the norm of a sublayer that this layer
    #: does not have): neither missed when absent nor refused when present, never drawn
    optional: bool = False

    def fits(self, shape) -> bool:
        shape = tuple(shape)
        return len(shape) == len(self.shape) and all(w is None or w == g for w, g in zip(self.shape, shape))


# --------------------------------------------------------------------------- cache needs


@dataclass(frozen=True)
class PagedTensorSpec:
    """One tensor that a mixer keeps per token, in pages.

    ``token_shape`` is what one token owns, for instance ``(kv_heads, head_dim)`` for a
    key. A page of ``page_size`` tokens has the token axis inserted at ``token_axis``:
    ``token_axis = 1`` on ``(kv_heads, head_dim)`` gives pages of ``(kv_heads, page_size,
    head_dim)`` (every head's keys of a page lie together), ``token_axis = 2`` gives
    ``(kv_heads, head_dim, page_size)`` (transposed: runs of tokens), ``token_axis = 0``
    gives ``(page_size, ...)`` (one record per token). The layout is the mixer's choice,
    made for its kernels; the cache manager only allocates what it is told.
    ``dtype`` is "model" (the engine's element type) or "float32".
    """

    name: str
    token_shape: tuple[int, ...]
    token_axis: int = 0
    dtype: str = "model"

    def __post_init__(self) -> None:
        if not (0 <= self.token_axis <= len(self.token_shape)):
            raise ValueError(f"paged tensor {self.name!r}: token_axis {self.token_axis} does not fit "
                             f"token_shape {self.token_shape}")
        if self.dtype not in ("model", "float32"):
            raise ValueError(f"paged tensor {self.name!r}: dtype must be 'model' or 'float32'")

    def page_shape(self, page_size: int) -> tuple[int, ...]:
        s = list(self.token_shape)
        s.insert(self.token_axis, page_size)
        return tuple(s)

    def elements_per_token(self) -> int:
        n = 1
        for d in self.token_shape:
            n *= d
        return n


@dataclass(frozen=True)
class PagedCacheSpec:
    """What a mixer keeps per token: one or more tensors in pages that share a block
    table. ``window`` = 0 keeps every token; ``window`` = W keeps the last W (a query at
    position p sees p-W+1 .. p), and pages that no later query can see are given back. ``chunk`` = C > 0:
    a query sees only the keys of its own run of C positions (runs counted from position 0), so the pages
    that lie wholly before the run of the next query are given back as well."""

    tensors: tuple[PagedTensorSpec, ...]
    window: int = 0
    #: with a window: the sequence's first ``keep_first`` tokens stay visible to every later query,
    #: so the pages that hold them are never given back
    keep_first: int = 0
    #: tokens per page that this mixer's kernels need, if they need a particular number; None:
    #: whatever the engine is set to. All page groups of an engine share one page size, so an
    #: engine set to another size refuses the model when it is built.
    page_size: int | None = None
    #: runs of this many positions: a query sees no key before its own run (0: no runs)
    chunk: int = 0

    kind: ClassVar[str] = "paged"

    def __post_init__(self) -> None:
        names = [t.name for t in self.tensors]
        if not names or len(names) != len(set(names)):
            raise ValueError("a paged cache needs at least one tensor, each with a name of its own")
        if self.window < 0 or self.keep_first < 0 or self.chunk < 0:
            raise ValueError("window, keep_first and chunk must not be negative")
        if self.page_size is not None and self.page_size <= 0:
            raise ValueError("page_size must be positive")


@dataclass(frozen=True)
class StateCacheSpec:
    """A fixed-size state per request: ``shape`` elements of ``dtype`` ("float32" or
    "model" for the engine's element type), zeroed when a request starts."""

    shape: tuple[int, ...]
    dtype: str = "float32"

    kind: ClassVar[str] = "state"


# --------------------------------------------------------------------------- the checkpoint's tensors at bind time


class TensorBag(dict):
    """The checkpoint's tensors while the parts take theirs. ``uses[name]`` counts the parts
    that named the tensor in their ``tensor_specs``; :func:`take` hands a tensor out and, when
    the last of them has come for it, drops it from the bag, so that a part which copies its
    tensors (a fused weight) does not keep the originals alive until the whole model is bound."""

    def __init__(self, tensors: dict, uses: dict[str, int]):
        super().__init__(tensors)
        self.uses = dict(uses)


def take(tensors: dict, name: str):
    """``tensors[name]``; out of the bag with it if nobody else is going to ask. With a plain
    dictionary this is ``tensors[name]`` and nothing more."""
    uses = getattr(tensors, "uses", None)
    if uses is None or name not in uses:
        return tensors[name]
    uses[name] -= 1
    return tensors.pop(name) if uses[name] <= 0 else tensors[name]


# --------------------------------------------------------------------------- part classes


@dataclass(frozen=True)
class StepArraySpec:
    """An int32 array that a part's kernels need of every step beside the common ones
    (tokens, positions, block tables, ...): work lists, tiles, anything that follows from
    the step's batch. ``build(host_batch)`` returns it (numpy int32, any shape);
    ``capacity(max_tokens, max_seqs)`` bounds its number of elements
    (``max_seqs`` as ``HostBatch.decode_shape`` rounds the number of single-token requests). The engine builds it
    on the host, uploads it in the step's one copy and hands it to the parts as
    ``ctx.arrays[name]`` (device) and ``ctx.host.arrays[name]`` (host). Parts that name the
    same array share it."""

    name: str
    capacity: Any = field(compare=False)
    build: Any = field(compare=False)


class Part:
    """Base of everything that owns tensors."""

    def tensor_specs(self) -> list[TensorSpec]:
        return []

    def linears(self) -> list:
        """The matrix products (:class:`~pyre_amd.parts.linear.Linear`) this part owns,
        for whoever wants to prepare them (the engine lets the BLAS library time its
        kernels for their shapes)."""
        return []

    def bind(self, tensors: dict[str, Any], runtime: Any) -> None:
        """Take the tensors named by ``tensor_specs`` out of ``tensors``."""


class Mixer(Part):
    def cache_spec(self) -> PagedCacheSpec | StateCacheSpec | None:
        return None

    def step_arrays(self) -> list[StepArraySpec]:
        """Arrays that this mixer's kernels want of every step beside the common ones."""
        return []

    def forward(self, ctx, h, cache):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, h):
        raise NotImplementedError


class Norm(Part):
    def forward(self, ctx, resid, delta, out, rows=None):
        raise NotImplementedError


class PositionEncoding(Part):
    def rotary(self, runtime):
        return None, None, 0


class Block(Part):
    """A layer: parts arranged around the residual stream. ``forward`` receives one cache view
    per description of ``cache_specs()``, in that order (or the views of the entry whose caches
    this call reads, ``LayerCall.cache_from``)."""

    def cache_specs(self) -> list:
        return []

    def step_arrays(self) -> list[StepArraySpec]:
        return []

    def forward(self, ctx, state, caches: list) -> None:
        raise NotImplementedError


# --------------------------------------------------------------------------- registry of parts

_PARTS: dict[tuple[str, str], type] = {}
ROLES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head", "token_input")


def register_part(role: str, kind: str, cls: type) -> None:
    if role not in ROLES:
        raise ValueError(f"unknown role {role!r}; roles are {ROLES}")
    _PARTS[(role, kind)] = cls


def make_part(role: str, spec: Any, **kw: Any):
    """Build the part that ``spec`` (a dataclass with a ``kind``) describes."""
    _load_builtin_parts()
    kind = getattr(spec, "kind", None)
    try:
        cls = _PARTS[(role, kind)]
    except KeyError:
        known = sorted(k for r, k in _PARTS if r == role)
        raise ValueError(f"no {role} of kind {kind!r} is registered; known: {known}") from None
    return cls(spec, **kw)


def _load_builtin_parts() -> None:
    import pyre_amd.parts.builtin  # noqa: F401


# --------------------------------------------------------------------------- descriptions


@dataclass(frozen=True)
class RMSNormSpec:
    hidden_size: int
    eps: float
    prefix: str                      #: tensor name is ``prefix + ".weight"``
    name: str | None = None          #: or this, as it stands
    one_plus: bool = False           #: the tensor is stored around zero: the gain is one plus it
    kind: ClassVar[str] = "rmsnorm"

    @property
    def tensor(self) -> str:
        return self.name if self.name is not None else f"{self.prefix}.weight"


@dataclass(frozen=True)
class RotarySpec:
    """Rotary positions: element j pairs with j + rotary_dim/2 (``pairing`` "halves"), or element 2j with 2j + 1
    ("neighbours": a mixer whose kernels turn such pairs says so); the angle of pair j is position * theta^(-2j/d)
    either way, so the tables are the same."""

    head_dim: int
    theta: float
    max_positions: int
    rotary_dim: int | None = None    #: None: the whole head
    #: angles position * theta^(-2j/d) formed in float64 and their cosines and sines rounded to float32 once,
    #: instead of float32 arithmetic all the way
    exact: bool = False
    pairing: str = "halves"
    #: (factor, original, fast, slow): the frequencies of pairs that turn fewer than ``slow`` times over ``original``
    #: positions are divided by ``factor``, those that turn more than ``fast`` times stay, those between are blended
    #: linearly by their index; cosines and sines are multiplied by 0.1 ln(factor) + 1. None: plain frequencies.
    scaling: tuple | None = None
    kind: ClassVar[str] = "rotary"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: ClassVar[str] = "none"


@dataclass(frozen=True)
class AttentionSpec:
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    position: Any                    #: a position-encoding description
    prefix: str                      #: e.g. "model.layers.0.self_attn"
    qkv_bias: bool = True
    out_bias: bool = False
    window: int = 0                  #: 0: every earlier key is visible
    scale: float | None = None       #: None: head_dim ** -0.5
    kind: ClassVar[str] = "attention"


@dataclass(frozen=True)
class LayerNormSpec:
    """(x - mean) / sqrt(var + eps) * gain, no bias; ``name`` is the gain's tensor."""

    hidden_size: int
    eps: float
    name: str
    kind: ClassVar[str] = "layernorm"


@dataclass(frozen=True)
class CappedAttentionSpec:
    """Softmax attention without rotation: unit-norm queries and keys (``unit_norm``), scores times
    ``scale``, squashed by ``softcap * tanh(s / softcap)`` (0: not), plus a learned bias by distance
    (``bias_rows`` rows of a table per head, one per distance below half of them, the rest spaced
    evenly in log(distance) up to ``bias_far``; None: the file says how many, 0: no bias), a window
    of ``window`` tokens (0: all) beside the sequence's first ``keep_first``, key heads of
    ``key_dim`` and value heads of ``value_dim`` elements, one sigmoid gate per head (``gated``).
    Tensors: ``prefix + .q / .k / .v / .g / .o / .rel``."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    prefix: str
    softcap: float = 0.0
    bias_far: float = 0.0
    bias_rows: int | None = None
    window: int = 0
    keep_first: int = 0
    unit_norm: bool = True
    norm_eps: float = 1e-6
    gated: bool = True
    kind: ClassVar[str] = "capped_attention"


@dataclass(frozen=True)
class GatedLinearAttentionSpec:
    """Per head a float32 state S [key_dim, value_dim]: S <- diag(a) S + k v^T, o = S^T q key_dim^-1/2,
    a = sigmoid(A2 (A1 h) + b)^(1 / tau) per key channel (``rank``: columns of A2; None: the file says).
    The heads' outputs are divided by their root mean square, times a gain over value_dim, times silu(G h).
    Tensors: ``prefix + .q / .k / .v / .g / .o / .norm / .a1 / .a2 / .a2.b``."""

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    tau: float
    prefix: str
    norm_eps: float = 1e-6
    rank: int | None = None
    kind: ClassVar[str] = "gated_linear_attention"


@dataclass(frozen=True)
class TanhNormSpec:
    """tanh(alpha x) * gain + shift, element by element: a norm that takes no statistic of the row. ``name`` is
    the gain's tensor; the scalar and the shift are ``name + ".alpha"`` and ``name + ".b"``."""

    hidden_size: int
    name: str
    kind: ClassVar[str] = "tanh_norm"


@dataclass(frozen=True)
class TiedAttentionSpec:
    """Grouped softmax attention whose values are its keys as projected (before any rotation): there is no value
    matrix. Scores times ``scale``; ``chunk`` = C > 0 lets a query see only the earlier keys of its own run of C
    positions (runs counted from position 0), 0 is plain causal attention. ``position`` describes the rotation of
    queries and keys (or none). Tensors: ``prefix + .q / .k / .o`` and, with ``bias``, ``.q.b / .k.b``."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: Any
    prefix: str
    chunk: int = 0
    bias: bool = True
    kind: ClassVar[str] = "tied_attention"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal softmax attention whose keys and values of all heads are made of one compressed row per token:
    c = rms_norm(Wdkv h) * gain [rank]; per head k = Wuk c (``key_dim``), v = Wuv c (``value_dim``). Only c is
    kept. ``own_latent`` False: the layer has no Wdkv and reads the rows that another layer keeps (the order of
    layers names it as the entry whose cache this one reads). Tensors: ``prefix + .q / .dkv / .dkv.norm / .uk /
    .uv / .o``."""

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    rank: int
    scale: float
    norm_eps: float
    prefix: str
    own_latent: bool = True
    kind: ClassVar[str] = "latent_attention"


@dataclass(frozen=True)
class GeluGLUSpec:
    """down(gelu_tanh(gate(x)) * up(x)), no biases. Tensors: ``prefix + .gate / .up / .down``."""

    hidden_size: int
    intermediate_size: int
    prefix: str
    kind: ClassVar[str] = "gelu_glu"


@dataclass(frozen=True)
class SigmoidMoESpec:
    """A mixture of ``experts`` feed-forward layers down(relu(up(x))^2) of ``expert_size`` hidden units each: every
    token goes through the ``top`` experts of largest sigmoid(router(x)), weighted by these scores over their sum
    (+ 1e-20); a shared expert of ``shared_size`` units (0: none) runs for every token and is added. Tensors:
    ``prefix + .router``, ``.e<i>.up / .down``, ``.shared.up / .down``."""

    hidden_size: int
    experts: int
    top: int
    expert_size: int
    prefix: str
    shared_size: int = 0
    kind: ClassVar[str] = "sigmoid_moe"


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped softmax attention over a window whose denominator holds one more term, exp(sink) of a learned number
    per head that has no key and no value (``sink``). Before anything else the projected queries, keys and values go
    through a causal convolution over time, ``conv_taps`` taps per channel (0: none), whose last ``conv_taps - 1``
    inputs a request keeps as state; queries and keys are then divided by their root mean square per head, times a
    gain over ``key_dim`` that the heads share (``qk_norm``), and turned by position (``position``: either pairing).
    The heads' outputs are multiplied element by element with sigmoid(G h) (``gated``). Tensors: ``prefix + .q / .k /
    .v / .g / .o / .sink / .q.norm / .k.norm / .q.conv / .k.conv / .v.conv``."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    position: Any
    prefix: str
    window: int = 0
    conv_taps: int = 0
    qk_norm: bool = True
    norm_eps: float = 1e-6
    sink: bool = True
    gated: bool = True
    kind: ClassVar[str] = "sink_attention"


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with one fixed decay per head: S <- decay_h S + k v^T, o = S^T q with S [key_dim, value_dim]
    float32 per head and request, no softmax and no denominator. Queries and keys are turned by position
    (``position``: either pairing), the keys then scaled by key_dim^-1/2. Every head's o is divided by its root mean
    square (no gain), times silu(G h). Tensors: ``prefix + .q / .k / .v / .g / .o``."""

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    decay: tuple
    position: Any
    prefix: str
    norm_eps: float = 1e-6
    kind: ClassVar[str] = "retention"


@dataclass(frozen=True)
class ReluSquaredMLPSpec:
    """down(relu(up(x))^2), no biases. Tensors: ``prefix + .up / .down``."""

    hidden_size: int
    intermediate_size: int
    prefix: str
    kind: ClassVar[str] = "relu2_mlp"


@dataclass(frozen=True)
class GroupedSoftmaxMoESpec:
    """A mixture of ``experts`` gated units down(silu(gate(x)) * up(x)) of ``expert_size`` hidden units and ``identity``
    further experts that hand their input back as it is (they own no tensors; the router's last outputs are theirs).
    Scores s = softmax(router(x)) over all of them; the choice goes by s + a learned correction per expert, among the
    experts of the ``keep_groups`` of ``groups`` equal groups of neighbours whose largest such number is largest; the
    ``top`` chosen experts are weighted by s itself, not renormalised. Tensors: ``prefix + .router / .correction``,
    ``.e<i>.gate / .up / .down``."""

    hidden_size: int
    experts: int
    top: int
    expert_size: int
    prefix: str
    identity: int = 0
    groups: int = 1
    keep_groups: int = 1
    kind: ClassVar[str] = "grouped_softmax_moe"


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Grouped softmax attention over a window of ``window`` tokens (0: all earlier ones) with biased projections
    (``qkv_bias``, ``out_bias``). ``wide_norm``: queries and keys are divided by their root mean square over their whole
    projection, all heads at once, times a gain over that projection, before they are turned by position (``position``,
    element e with e + rot/2). ``sink``: "zero" adds one term of score 0, without a value, to the softmax's denominator;
    "none" is the ordinary softmax. ``own_kv`` False: the layer has no key and value projections and reads the pages that
    another layer keeps (the order of layers names it). ``cache_window``: the window by which pages are given back, if it
    has to be wider than the layer's own (a layer whose pages another reads with a wider window; 0 with a window of its
    own: never). Tensors: ``prefix + .q / .k / .v / .o`` with ``.b`` for the biases, ``.q.norm / .k.norm``."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    position: Any
    prefix: str
    window: int = 0
    qkv_bias: bool = True
    out_bias: bool = False
    wide_norm: bool = False
    norm_eps: float = 1e-6
    sink: str = "none"
    own_kv: bool = True
    cache_window: int | None = None
    kind: ClassVar[str] = "window_attention"


@dataclass(frozen=True)
class GatedDeltaRuleSpec:
    """Per value head a float32 state S [key_dim, value_dim]: S <- diag(a) S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q. ``num_kv_heads`` query/key heads serve ``num_heads`` value heads. q, k and v go through a short causal
    convolution (``conv_taps`` per channel, no bias) and SiLU; q and k are then unit vectors per head (``unit_eps`` beside
    the sum of squares), q times key_dim^-1/2. beta = sigmoid(B h); a = exp(-exp(A_log_h) softplus(A2 (A1 h) + dt_bias))
    per head and key channel; every head's o is divided by its root mean square (``norm_eps``), times a gain over
    value_dim, times sigmoid(G2 (G1 h)). The ranks of the two low-rank products are the file's to say (None).
    Tensors: ``prefix + .q / .k / .v / .b / .a1 / .a2 / .g1 / .g2 / .o / .q.conv / .k.conv / .v.conv / .A_log /
    .dt_bias / .norm``."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    conv_taps: int
    prefix: str
    norm_eps: float = 1e-6
    unit_eps: float = 1e-6
    decay_rank: int | None = None
    gate_rank: int | None = None
    kind: ClassVar[str] = "gated_delta_rule"


@dataclass(frozen=True)
class SoftmaxTopKMoESpec:
    """A mixture of ``experts`` gated units down(silu(gate(x)) * up(x)) of ``expert_size`` hidden units: every token goes
    through the ``top`` experts of largest router logit (``router_bias``: the router has a bias), weighted by the softmax
    over the chosen logits alone; a shared expert of ``shared_size`` units (0: none) runs for every token and is added,
    times sigmoid(sg . x), one number per token (``shared_gate``). Tensors: ``prefix + .router / .router.b``,
    ``.e<i>.gate / .up / .down``, ``.shared.gate / .up / .down / .sg``."""

    hidden_size: int
    experts: int
    top: int
    expert_size: int
    prefix: str
    shared_size: int = 0
    shared_gate: bool = True
    router_bias: bool = True
    kind: ClassVar[str] = "softmax_topk_moe"


@dataclass(frozen=True)
class TokenSideSpec:
    """A layer's input from the token itself: proj(gelu_tanh(gate(x)) * table[token, first : first + dim]), x the residual
    stream. ``table`` is shared by the layers, each of which takes ``dim`` of its ``table_width`` columns. Tensors: ``table``,
    ``prefix + .gate / .proj``."""

    hidden_size: int
    vocab_size: int
    dim: int
    table: str
    table_width: int
    first: int
    prefix: str
    kind: ClassVar[str] = "token_side"


@dataclass(frozen=True)
class PostNormBlockSpec:
    """x += post_norm(mixer(x)); x += post_norm(feed_forward(x)): the sublayers read the residual stream itself (in the
    engine's element type) and only their results are normed (RMS norms). ``feed_forward`` None: the first half alone."""

    mixer: Any
    mixer_post_norm: Any
    feed_forward: Any = None
    feed_forward_post_norm: Any = None
    kind: ClassVar[str] = "post_norm"


@dataclass(frozen=True)
class ParallelBlockSpec:
    """x += scale * (mixer(norm(x)) + feed_forward(norm(x))): one norm, both sublayers read its rows
    (``feed_forward`` None: the mixer alone)."""

    mixer: Any
    norm: Any
    feed_forward: Any = None
    scale: float = 1.0
    kind: ClassVar[str] = "parallel_block"


@dataclass(frozen=True)
class ParallelMixerSpec:
    """sum_i scales[i] * branches[i](h): mixers side by side that read the same rows. ``out_norms``: every branch's
    result is first divided by its root mean square over the hidden size (``norm_eps``), times a gain of its own
    (the tensors named here, one per branch); the branches then keep their output products apart."""

    hidden_size: int
    branches: tuple
    scales: tuple
    out_norms: tuple | None = None
    norm_eps: float = 1e-6
    kind: ClassVar[str] = "parallel"


@dataclass(frozen=True)
class ClippedGLUSpec:
    """down(g sigmoid(slope g) (u + 1)), g = min(gate(x), limit), u = clamp(up(x), -limit, limit).
    Tensors: ``prefix + .gate / .up / .down``."""

    hidden_size: int
    intermediate_size: int
    limit: float
    prefix: str
    slope: float = 1.702
    kind: ClassVar[str] = "clipped_glu"


@dataclass(frozen=True)
class SandwichBlockSpec:
    """x += mixer_scale * mixer_post_norm(mixer(mixer_norm(x))), then the same around the
    feed-forward (None: the layer has none). The scales are tensors over the hidden size."""

    mixer: Any
    mixer_norm: Any
    mixer_post_norm: Any
    mixer_scale: str | None
    feed_forward: Any = None
    feed_forward_norm: Any = None
    feed_forward_post_norm: Any = None
    feed_forward_scale: str | None = None
    #: tensors over the hidden size that a file may hold for this layer though nothing reads them
    unused: tuple = ()
    kind: ClassVar[str] = "sandwich"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden_size: int
    intermediate_size: int
    prefix: str                      #: e.g. "model.layers.0.mlp"
    kind: ClassVar[str] = "swiglu"


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(norm(x)); x += feed_forward(norm(x))   (pre-norm residual block; ``feed_forward`` None: the first half
    alone). ``token_input``: a third sublayer that reads the residual stream itself and the step's tokens, whose result is
    RMS-normed (``token_input_norm``) before it joins the stream."""

    mixer: Any
    mixer_norm: Any
    feed_forward: Any
    feed_forward_norm: Any
    token_input: Any = None
    token_input_norm: Any = None
    kind: ClassVar[str] = "pre_norm"


@dataclass(frozen=True)
class EmbeddingSpec:
    vocab_size: int
    hidden_size: int
    name: str = "model.embed_tokens.weight"
    scale: float = 1.0               #: the table's rows are multiplied by this
    kind: ClassVar[str] = "embedding"


@dataclass(frozen=True)
class BigramEmbeddingSpec:
    """table[token] + pairs[(previous token * mul_prev + token * mul_cur) mod buckets]; a request's first token
    takes row ``buckets`` of ``pairs`` (its last). The previous token is state that a request keeps."""

    vocab_size: int
    hidden_size: int
    buckets: int
    mul_prev: int
    mul_cur: int
    name: str = "embed"
    pairs_name: str = "bigram"
    kind: ClassVar[str] = "bigram_embedding"


@dataclass(frozen=True)
class LMHeadSpec:
    vocab_size: int
    hidden_size: int
    name: str = "lm_head.weight"
    tied_to: str | None = None       #: embedding tensor used when the head is tied
    scale: float = 1.0               #: the logits are multiplied by this
    softcap: float = 0.0             #: c > 0: then squashed, c * tanh(logit / c)
    kind: ClassVar[str] = "lm_head"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the order in which layers run.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named more than once).
    ``cache_from`` = j lets this call's mixer read the cache that the j-th entry
    of the order wrote, instead of keeping one of its own.
    """

    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: Any
    layers: tuple[Any, ...]
    schedule: tuple[LayerCall, ...]
    final_norm: Any
    head: Any
    extra: dict = field(default_factory=dict, compare=False)
