"""Mixers whose matrix products can be shared: several of them side by side read the same rows,
so their input products are one product over the row-wise concatenation of their matrices, and
their scaled results are one output product over the column-wise concatenation of theirs."""

from __future__ import annotations

import torch

from pyre_amd.hip.ops import Partials, PostNorm
from pyre_amd.parts.base import Mixer, ParallelMixerSpec, TensorSpec, make_part, take
from pyre_amd.parts.linear import Linear


#: columns of a shared input product at which a branch's own begin
COLUMN_ALIGN = 8


class BranchMixer(Mixer):
    """A mixer of the form out(f(in_1 h, in_2 h, ...)): all its input matrices multiply the rows it is
    given, and one output matrix multiplies what it makes of them. It says which matrices these are
    and does the part in between (``attend``); the products are run here when it stands alone, or by a
    :class:`ParallelMixer` for all its branches at once.

    A subclass provides ``hidden_size``, ``inner`` (columns of the rows that ``attend`` writes),
    ``in_tensors()`` (the input matrices in the order of the product's columns), ``out_tensor()``,
    ``other_tensors()`` / ``bind_others()`` for what else it owns, and
    ``attend(ctx, proj, col0, cache, o, scale)``: from the input product's partial sums (its own
    columns start at ``col0``) to ``o [n, inner]`` (rows ``o.stride(0)`` apart), times ``scale``."""

    hidden_size: int
    inner: int
    role = "mix"

    def in_tensors(self) -> list[TensorSpec]:
        raise NotImplementedError

    def out_tensor(self) -> TensorSpec:
        raise NotImplementedError

    def in_biases(self) -> list:
        """One entry per input matrix, in their order: the description of its bias, or None. A product with biases hands
        them on as its pending bias (float32 over all its columns); ``attend`` must then be one that adds it."""
        return [None] * len(self.in_tensors())

    def out_bias(self) -> TensorSpec | None:
        return None

    def other_tensors(self) -> list[TensorSpec]:
        return []

    def bind_others(self, tensors, runtime) -> None:
        pass

    def attend(self, ctx, proj: Partials, col0: int, cache, o: torch.Tensor, scale: float) -> None:
        raise NotImplementedError

    def cache_specs(self) -> list:
        """What the mixer keeps, one description per cache (a mixer with pages and a state of its own has two);
        ``attend`` gets the one view, or the list of them if there are several."""
        spec = self.cache_spec()
        return [] if spec is None else [spec]

    # ---- standing alone
    def tensor_specs(self) -> list[TensorSpec]:
        return [*self.in_tensors(), self.out_tensor(), *_bias_specs(self), *self.other_tensors()]

    def bind(self, tensors, runtime) -> None:
        bias = _in_bias(self, tensors)
        w = _stacked([s.name for s in self.in_tensors()], tensors, 0)  # a size that only the file knows is known now
        pad = -w.shape[0] % COLUMN_ALIGN
        if pad:
            # rows of zeros behind a product whose width is no multiple of eight: its rows then start on 16 bytes,
            # which the kernels that finish it four columns at a time need
            w = torch.cat([w, torch.zeros(pad, w.shape[1], dtype=w.dtype, device=w.device)], dim=0)
            if bias is not None:
                bias.append(torch.zeros(pad, dtype=torch.float32, device=w.device))
        self._in = Linear(self.hidden_size, w.shape[0], f"{self.role}.in")
        self._out = Linear(self.inner, self.hidden_size, f"{self.role}.out")
        self._in.set(w, None if bias is None else torch.cat(bias))
        ob = self.out_bias()
        self._out.set(take(tensors, self.out_tensor().name), None if ob is None else take(tensors, ob.name).float())
        self.bind_others(tensors, runtime)

    def linears(self) -> list:
        return [self._in, self._out]

    def forward(self, ctx, h, cache):
        n = ctx.n_tokens
        proj = self._in.forward(ctx, h, n)
        o = ctx.workspace.get(f"{self.role}.o", (n, self.inner), ctx.dtype)
        if isinstance(cache, (list, tuple)) and len(self.cache_specs()) <= 1:  # a block that hands over all its views
            cache = cache[0] if cache else None
        self.attend(ctx, proj, 0, cache, o, 1.0)
        return self._out.forward(ctx, o, n)


def _bias_specs(b) -> list[TensorSpec]:
    return [s for s in (*b.in_biases(), b.out_bias()) if s is not None]


def _in_bias(b, tensors):
    """The biases of a branch's input matrices as float32 pieces in the order of the product's columns (zeros where a
    matrix has none), or None if no matrix has one. Called before the matrices are taken out of the bag."""
    specs, biases = b.in_tensors(), b.in_biases()
    if all(x is None for x in biases):
        return None
    out = []
    for spec, bias in zip(specs, biases):
        w = tensors[spec.name]
        out.append(take(tensors, bias.name).float() if bias is not None
                   else torch.zeros(w.shape[0], dtype=torch.float32, device=w.device))
    return out


def _stacked(names, tensors, dim):
    """The named tensors concatenated along ``dim``, each let go of as soon as it is copied."""
    parts = [take(tensors, n) for n in names]
    if len(parts) == 1:
        return parts[0]
    fused = torch.cat(parts, dim=dim)
    del parts
    return fused


class ParallelMixer(Mixer):
    """sum_i scale_i * branch_i(h). One input product for all branches, one output product over
    [scale_0 o_0 | scale_1 o_1 | ...] against [Wo_0 | Wo_1 | ...]; every branch keeps its own caches
    (``cache_specs``: the branches' descriptions in their order).

    With ``out_norms`` every branch's result is normed over the hidden size before the sum, so the output products
    stay apart (one per branch); none of the norms runs here: the results are handed on as pending terms, each with
    its norm and factor, and the kernel that adds them to the residual stream applies both."""

    def __init__(self, spec: ParallelMixerSpec):
        if len(spec.branches) != len(spec.scales) or not spec.branches:
            raise ValueError("parallel mixer: one scale per branch, at least one branch")
        self.spec = spec
        self.branches = [make_part("mixer", b) for b in spec.branches]
        for b in self.branches:
            if not isinstance(b, BranchMixer):
                raise ValueError(f"parallel mixer: {type(b).__name__} cannot share its products")
        if spec.out_norms is not None and (len(spec.out_norms) != len(spec.branches) or len(spec.branches) > 2):
            raise ValueError("parallel mixer: one output norm per branch, and at most two branches that are normed apart")
        self.inner = sum(b.inner for b in self.branches)
        self.proj = self.out = None   # made when the tensors are bound: a size may be the file's to say
        self.outs: list[Linear] = []  # with out_norms: one output product per branch
        self.out_gains: list[torch.Tensor] = []
        self.first_column: list[int] = []

    def cache_specs(self) -> list:
        return [s for b in self.branches for s in b.cache_specs()]

    def step_arrays(self) -> list:
        return [a for b in self.branches for a in b.step_arrays()]

    def tensor_specs(self) -> list[TensorSpec]:
        norms = [TensorSpec(n, (self.spec.hidden_size,), init="gain") for n in (self.spec.out_norms or ())]
        return [s for b in self.branches for s in (*b.in_tensors(), b.out_tensor(), *_bias_specs(b), *b.other_tensors())] + norms

    def bind(self, tensors, runtime) -> None:
        # every branch's columns start at a multiple of eight (rows of zeros between them), so that the
        # kernels which finish the product read them in 16-byte pieces
        col, parts, biases = 0, [], []
        self.first_column = []
        for b in self.branches:
            self.first_column.append(col)
            bias = _in_bias(b, tensors)
            mine = [take(tensors, s.name) for s in b.in_tensors()]
            rows = sum(t.shape[0] for t in mine)
            pad = -rows % COLUMN_ALIGN   # (behind the last branch too: the product's rows then start on 16 bytes)
            if pad:
                mine.append(torch.zeros(pad, mine[0].shape[1], dtype=mine[0].dtype, device=mine[0].device))
                rows += pad
            biases.append(bias if bias is None else torch.cat(bias + [torch.zeros(rows - sum(x.numel() for x in bias),
                                                                                  dtype=torch.float32, device=mine[0].device)]))
            parts += mine
            col += rows
        self.proj = Linear(self.spec.hidden_size, col, "mix.in")
        bias = None
        if any(x is not None for x in biases):  # one bias over all branches' columns, zero where a branch has none
            rows = [*self.first_column[1:], col]
            bias = torch.cat([x if x is not None else torch.zeros(rows[i] - self.first_column[i], dtype=torch.float32,
                                                                  device=parts[0].device) for i, x in enumerate(biases)])
        self.proj.set(torch.cat(parts, dim=0), bias)
        del parts, mine
        if self.spec.out_norms is None:
            self.out = Linear(self.inner, self.spec.hidden_size, "mix.out")
            # the sum of the branches' output biases, each times its branch's factor
            out_bias = None
            for b, scale in zip(self.branches, self.spec.scales):
                ob = b.out_bias()
                if ob is not None:
                    term = take(tensors, ob.name).float() * float(scale)
                    out_bias = term if out_bias is None else out_bias + term
            self.out.set(_stacked([b.out_tensor().name for b in self.branches], tensors, 1), out_bias)
        else:
            for i, (b, name) in enumerate(zip(self.branches, self.spec.out_norms)):
                if b.out_bias() is not None:
                    raise ValueError("parallel mixer: branches that are normed apart have no output bias")
                lin = Linear(b.inner, self.spec.hidden_size, f"mix.out{i}")
                lin.set(take(tensors, b.out_tensor().name))
                self.outs.append(lin)
                self.out_gains.append(take(tensors, name).contiguous())
        for b in self.branches:
            b.bind_others(tensors, runtime)

    def linears(self) -> list:
        return [self.proj, *([self.out] if self.out is not None else self.outs)]

    def forward(self, ctx, h, caches):
        n = ctx.n_tokens
        proj = self.proj.forward(ctx, h, n)
        apart = self.spec.out_norms is not None
        o = None if apart else ctx.workspace.get("mix.o", (n, self.inner), ctx.dtype)
        views = iter(caches or [])
        at = 0
        terms = []
        for i, (b, scale, col) in enumerate(zip(self.branches, self.spec.scales, self.first_column)):
            mine = [next(views) for _ in b.cache_specs()]
            cache = mine[0] if len(mine) == 1 else (mine or None)
            if not apart:
                b.attend(ctx, proj, col, cache, o[:, at:at + b.inner], float(scale))
                at += b.inner
                continue
            # the branch's own rows, output product and norm; its factor rides on the pending term
            rows = ctx.workspace.get(f"mix.o{i}", (n, b.inner), ctx.dtype)
            b.attend(ctx, proj, col, cache, rows, 1.0)
            p = self.outs[i].forward(ctx, rows, n)
            terms.append(Partials(p.data, p.bias, PostNorm(self.out_gains[i], self.spec.norm_eps, kind="rms"), float(scale)))
        if not apart:
            return self.out.forward(ctx, o, n)
        for first, second in zip(terms, terms[1:]):
            first.more = second
        return terms[0]
