"""The arrangement of a layer's parts around the residual stream (`pyre/model.py:142-153`)."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from pyre_amd.hip.ops import Partials, PostNorm
from pyre_amd.parts.base import (Block, BlockSpec, ParallelBlockSpec, PostNormBlockSpec, SandwichBlockSpec, TensorSpec,
                                 make_part, take)


@dataclass
class Hidden:
    """The residual stream (float32 [N, H]) and the term not yet added to it: the
    next norm adds it in the same kernel that norms the sum."""

    resid: torch.Tensor
    pending: Partials | None = None


class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)), the second half only if the layer has a feed-forward. A layer
    may have a third sublayer that reads the residual stream itself and the step's tokens (``token_input``): the kernel
    that adds the pending term also writes the stream's rows in the engine's element type for it, and its result is
    handed on with its RMS norm, which the next norm's kernel applies as it adds. A mixer made of several
    (``cache_specs`` on the mixer) gets all of the block's cache views, a plain one its own."""

    def __init__(self, spec: BlockSpec):
        self.spec = spec
        self.mixer = make_part("mixer", spec.mixer)
        self.mixer_norm = make_part("norm", spec.mixer_norm)
        self.feed_forward = self.feed_forward_norm = self.token_input = self.token_input_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = make_part("feed_forward", spec.feed_forward)
            self.feed_forward_norm = make_part("norm", spec.feed_forward_norm)
        if spec.token_input is not None:
            self.token_input = make_part("token_input", spec.token_input)
            self.token_input_norm = make_part("norm", spec.token_input_norm)

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward,
                                 self.token_input, self.token_input_norm) if p is not None)

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)
        if self.token_input_norm is not None and self.mixer_norm.gain.dtype == torch.float32:
            # the kernel that adds a normed term and norms the sum takes one element type for all its gains
            self.token_input_norm.gain = self.token_input_norm.gain.float().contiguous()

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def cache_specs(self) -> list:
        if hasattr(self.mixer, "cache_specs"):
            return list(self.mixer.cache_specs())
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def step_arrays(self) -> list:
        return self.mixer.step_arrays()

    def forward(self, ctx, state: Hidden, caches: list) -> None:
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        self.mixer_norm.forward(ctx, state.resid, state.pending, h)
        cache = caches if hasattr(self.mixer, "cache_specs") else (caches[0] if caches else None)
        state.pending = self.mixer.forward(ctx, h, cache)
        if self.feed_forward is not None:
            self.feed_forward_norm.forward(ctx, state.resid, state.pending, h)
            state.pending = self.feed_forward.forward(ctx, h)
        if self.token_input is None:
            return
        from pyre_amd.hip import ops

        pending = state.pending
        if pending is not None and pending.bias is not None:  # the kernel below takes no pending bias: summed first
            full = ctx.workspace.get("block.sum", (1, ctx.n_tokens, state.resid.shape[1]), torch.float32)
            ops.reduce_partials(pending, full[0], ctx.n_tokens)
            pending = Partials(full)
        ops.add_rms_terms(state.resid, pending, None, 0.0, h)   # the pending term joins the stream; h = the stream
        term = self.token_input.forward(ctx, h)
        norm = self.token_input_norm
        state.pending = Partials(term.data, term.bias, PostNorm(norm.gain, norm.spec.eps, kind="rms"))


class SandwichBlock(Block):
    """x += s1 * post1(mixer(norm1(x))); x += s2 * post2(feed_forward(norm2(x))): every sublayer is
    normed before and after, and its normed result is scaled element by element before it is added.
    The post-norms never run as kernels of their own: a sublayer's result is handed on as the pending
    term together with its norm and scale, and the next norm's kernel applies them as it adds. A layer
    without a feed-forward is the first half alone. A mixer made of several (``cache_specs`` on the
    mixer) gets all of the block's cache views, a plain one its own."""

    def __init__(self, spec: SandwichBlockSpec):
        self.spec = spec
        self.mixer = make_part("mixer", spec.mixer)
        self.mixer_norm = make_part("norm", spec.mixer_norm)
        self.mixer_post = make_part("norm", spec.mixer_post_norm)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_post = None
        if spec.feed_forward is not None:
            self.feed_forward = make_part("feed_forward", spec.feed_forward)
            self.feed_forward_norm = make_part("norm", spec.feed_forward_norm)
            self.feed_forward_post = make_part("norm", spec.feed_forward_post_norm)
        self.scales: dict[str, torch.Tensor] = {}

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.feed_forward_norm,
                                 self.feed_forward, self.feed_forward_post) if p is not None)

    def _scale_names(self):
        return [n for n in (self.spec.mixer_scale, self.spec.feed_forward_scale if self.feed_forward else None) if n]

    def tensor_specs(self) -> list[TensorSpec]:
        hidden = self.mixer_norm.spec.hidden_size
        return [s for p in self.parts() for s in p.tensor_specs()] + \
               [TensorSpec(n, (hidden,), init="gain") for n in self._scale_names()] + \
               [TensorSpec(n, (hidden,), init="gain", optional=True) for n in self.spec.unused]

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)
        for n in self._scale_names():
            self.scales[n] = take(tensors, n).contiguous()
        for n in self.spec.unused:
            if n in tensors:
                take(tensors, n)

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def cache_specs(self) -> list:
        if hasattr(self.mixer, "cache_specs"):
            return list(self.mixer.cache_specs())
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def step_arrays(self) -> list:
        return self.mixer.step_arrays()

    def _post(self, term: Partials, norm, scale_name) -> Partials:
        if term.post is not None:
            raise ValueError("a sublayer's result already carries a norm")
        return Partials(term.data, term.bias, PostNorm(norm.gain, norm.spec.eps, self.scales.get(scale_name)))

    def forward(self, ctx, state: Hidden, caches: list) -> None:
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        self.mixer_norm.forward(ctx, state.resid, state.pending, h)
        cache = caches if hasattr(self.mixer, "cache_specs") else (caches[0] if caches else None)
        state.pending = self._post(self.mixer.forward(ctx, h, cache), self.mixer_post, self.spec.mixer_scale)
        if self.feed_forward is None:
            return
        self.feed_forward_norm.forward(ctx, state.resid, state.pending, h)
        state.pending = self._post(self.feed_forward.forward(ctx, h), self.feed_forward_post,
                                   self.spec.feed_forward_scale)


class ParallelBlock(Block):
    """x += scale * (mixer(norm(x)) + feed_forward(norm(x))): one norm whose rows both sublayers read. Neither
    result is added here: both are handed on as the pending term (the second as ``Partials.more``, each with the
    factor), and the next norm's kernel adds them to the residual stream as it norms."""

    def __init__(self, spec: ParallelBlockSpec):
        self.spec = spec
        self.norm = make_part("norm", spec.norm)
        self.mixer = make_part("mixer", spec.mixer)
        self.feed_forward = make_part("feed_forward", spec.feed_forward) if spec.feed_forward is not None else None

    def parts(self):
        return tuple(p for p in (self.norm, self.mixer, self.feed_forward) if p is not None)

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def cache_specs(self) -> list:
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def step_arrays(self) -> list:
        return self.mixer.step_arrays()

    def forward(self, ctx, state: Hidden, caches: list) -> None:
        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        self.norm.forward(ctx, state.resid, state.pending, h)
        mixed = self.mixer.forward(ctx, h, caches[0] if caches else None)
        if mixed.post is not None or mixed.more is not None or mixed.scale != 1.0:
            raise ValueError("a parallel block takes a sublayer's plain result")
        more = None
        if self.feed_forward is not None:
            fed = self.feed_forward.forward(ctx, h)
            more = Partials(fed.data, fed.bias, scale=self.spec.scale)
        state.pending = Partials(mixed.data, mixed.bias, scale=self.spec.scale, more=more)


class PostNormBlock(Block):
    """x += post1(mixer(x)); x += post2(feed_forward(x)) with RMS norms: the sublayers read the residual stream itself,
    rounded to the engine's element type, and only what they return is normed. No norm runs as a kernel of its own: a
    sublayer's result is handed on as the pending term with its norm (``Partials.outer``: the norm of the sum of the
    term's parts, which a mixer of several branches may have normed and scaled one by one), and the kernel that adds
    it also writes the rows that the next sublayer reads. A layer without a feed-forward is the first half alone."""

    def __init__(self, spec: PostNormBlockSpec):
        self.spec = spec
        self.mixer = make_part("mixer", spec.mixer)
        self.mixer_post = make_part("norm", spec.mixer_post_norm)
        self.feed_forward = self.feed_forward_post = None
        if spec.feed_forward is not None:
            self.feed_forward = make_part("feed_forward", spec.feed_forward)
            self.feed_forward_post = make_part("norm", spec.feed_forward_post_norm)

    def parts(self):
        return tuple(p for p in (self.mixer, self.mixer_post, self.feed_forward, self.feed_forward_post) if p is not None)

    def tensor_specs(self) -> list[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, runtime) -> None:
        for p in self.parts():
            p.bind(tensors, runtime)

    def linears(self) -> list:
        return [lin for p in self.parts() for lin in p.linears()]

    def cache_specs(self) -> list:
        if hasattr(self.mixer, "cache_specs"):
            return list(self.mixer.cache_specs())
        spec = self.mixer.cache_spec()
        return [] if spec is None else [spec]

    def step_arrays(self) -> list:
        return self.mixer.step_arrays()

    @staticmethod
    def _post(term: Partials, norm) -> Partials:
        if term.outer is not None:
            raise ValueError("a sublayer's result already carries a norm of its sum")
        return Partials(term.data, term.bias, term.post, term.scale, term.more, PostNorm(norm.gain, norm.spec.eps, kind="rms"))

    def forward(self, ctx, state: Hidden, caches: list) -> None:
        from pyre_amd.hip import ops

        h = ctx.workspace.get("block.h", (ctx.n_tokens, state.resid.shape[1]), ctx.dtype)
        ops.add_rms_terms(state.resid, state.pending, None, 0.0, h)   # the pending term joins the stream; h = the stream
        cache = caches if hasattr(self.mixer, "cache_specs") else (caches[0] if caches else None)
        state.pending = self._post(self.mixer.forward(ctx, h, cache), self.mixer_post)
        if self.feed_forward is None:
            return
        ops.add_rms_terms(state.resid, state.pending, None, 0.0, h)
        state.pending = self._post(self.feed_forward.forward(ctx, h), self.feed_forward_post)
