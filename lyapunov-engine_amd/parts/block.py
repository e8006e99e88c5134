"""Arrangements of a layer's parts around the residual stream.

"prenorm" is the reference's decoder layer
(python/lyapunov_engine/models/llama.py:125-165): h += mixer(norm1(h));
h += ffn(norm2(h)).  The adds are carried out by the norm that follows them (see
parts/base.py), so the block returns the feed-forward's output still to be
added.
"""
from __future__ import annotations

import torch

from ..config.registry import BLOCKS, FEED_FORWARDS, FILTERS, MIXERS, NORMS
from ..config.specs import LayerSpec
from ..kernels import ops
from .base import Block, LayerCache, StepContext, WeightSource, WeightSpec


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.norm2 = NORMS.build(spec.norm2)
        self.ffn = FEED_FORWARDS.build(spec.ffn)

    def children(self):
        n = self.names
        return {n["norm1"] + ".": self.norm1, n["mixer"] + ".": self.mixer, n["norm2"] + ".": self.norm2,
                n["ffn"] + ".": self.ffn}

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        x = normed(self.norm1, self.mixer, ctx, h, delta)
        a = self.mixer.forward(ctx, x, cache)
        x = normed(self.norm2, self.ffn, ctx, h, a)
        return h, self.ffn.forward(ctx, x)


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """A norm in front of and behind each branch, a multiplier on what joins,
    and optionally a filter over time on what the mixer reads:

        h += mult * norm1_out(mixer(filter(norm1(h))));  h += mult * norm2_out(ffn(norm2(h)))

    The feed-forward branch may be absent (``LayerSpec.ffn`` None).  The further
    parts come from ``LayerSpec.extra``: "norm1_out", "norm2_out" (norms) and
    "filter" (an input filter); ``LayerSpec.params["mult"]`` is the multiplier.
    A branch's join is carried out by the norm that follows it, in one kernel
    (ops.JoiningBranch); the block returns its last branch still to be joined."""

    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.mult = float(spec.params.get("mult", 1.0))
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.norm1_out = NORMS.build(spec.extra["norm1_out"])
        self.filter = FILTERS.build(spec.extra["filter"]) if "filter" in spec.extra else None
        self.ffn = FEED_FORWARDS.build(spec.ffn) if spec.ffn is not None else None
        self.norm2 = NORMS.build(spec.norm2) if self.ffn is not None else None
        self.norm2_out = NORMS.build(spec.extra["norm2_out"]) if self.ffn is not None else None
        unknown = set(spec.extra) - {"norm1_out", "norm2_out", "filter"}
        if unknown:
            raise ValueError(f"the sandwich arrangement has no parts {sorted(unknown)}")

    def children(self):
        n = self.names
        out = {n["norm1"]: self.norm1, n["mixer"]: self.mixer, n["norm1_out"]: self.norm1_out}
        if self.filter is not None:
            out[n["filter"]] = self.filter
        if self.ffn is not None:
            out.update({n["norm2"]: self.norm2, n["ffn"]: self.ffn, n["norm2_out"]: self.norm2_out})
        return out

    def state_specs(self):
        out = super().state_specs()
        st = self.filter.state_spec() if self.filter is not None else None
        if st is not None:
            out["filter"] = st
        return out

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        conv = None
        if self.filter is not None and ctx.T == ctx.B and (delta is None or isinstance(delta, ops.JoiningBranch)) \
                and getattr(self.norm1, "joins_branches", False):
            # every request brings one token: the filter rides in the norm's kernel
            conv = self.filter.fused(ctx, cache.states.get("filter"), self.norm1.size)
        if conv is not None:
            x = self.norm1.forward(ctx, h, delta, conv=conv)
        else:
            x = normed(self.norm1, None, ctx, h, delta)
            if self.filter is not None:
                x = self.filter.forward(ctx, x, cache.states.get("filter"))
        branch = self.norm1_out.branch(self.mixer.forward(ctx, x, cache), self.mult)
        if self.ffn is None:
            return h, branch
        x = self.norm2.forward(ctx, h, branch)
        return h, self.norm2_out.branch(self.ffn.forward(ctx, x), self.mult)


@BLOCKS.register("prenorm_scaled")
class ScaledPreNormBlock(Block):
    """The pre-norm arrangement with a learned vector on what each branch adds, and optionally a
    filter over time on what the mixer reads:

        h += s1 * mixer(filter(norm1(h)));  h += s2 * ffn(norm2(h))

    s1 and s2 are tensors of the layer itself (``names["scale1"]``, ``names["scale2"]``); the filter
    comes from ``LayerSpec.extra["filter"]``.  The feed-forward branch may be absent.  A branch's
    product with its vector and the sum are carried out by the norm that follows (one with
    ``takes_scaled``, through an ``ops.ScaledBranch``); the block returns its last branch still to
    be added."""

    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.filter = FILTERS.build(spec.extra["filter"]) if "filter" in spec.extra else None
        self.ffn = FEED_FORWARDS.build(spec.ffn) if spec.ffn is not None else None
        self.norm2 = NORMS.build(spec.norm2) if self.ffn is not None else None
        self.hidden_size = int(spec.params["hidden_size"])
        self.scale1 = self.scale2 = None
        self.scale1_f = self.scale2_f = None
        unknown = set(spec.extra) - {"filter"}
        if unknown:
            raise ValueError(f"the scaled pre-norm arrangement has no parts {sorted(unknown)}")

    def weight_specs(self):
        n, shape = self.names, (self.hidden_size,)
        specs = [WeightSpec("scale1", (WeightSource(n["scale1"], shape),), init="ones")]
        if self.ffn is not None:
            specs.append(WeightSpec("scale2", (WeightSource(n["scale2"], shape),), init="ones"))
        return specs

    def children(self):
        n = self.names
        out = {n["norm1"]: self.norm1, n["mixer"]: self.mixer}
        if self.filter is not None:
            out[n["filter"]] = self.filter
        if self.ffn is not None:
            out.update({n["norm2"]: self.norm2, n["ffn"]: self.ffn})
        return out

    def materialize(self, device, dtype):
        super().materialize(device, dtype)
        self.scale1_f = self.scale1.float().contiguous()
        if self.scale2 is not None:
            self.scale2_f = self.scale2.float().contiguous()

    def state_specs(self):
        out = super().state_specs()
        st = self.filter.state_spec() if self.filter is not None else None
        if st is not None:
            out["filter"] = st
        return out

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        x = normed(self.norm1, None, ctx, h, delta)
        if self.filter is not None:
            x = self.filter.forward(ctx, x, cache.states.get("filter"))
        branch = ops.ScaledBranch(self.mixer.forward(ctx, x, cache), self.scale1_f)
        if self.ffn is None:
            return h, branch
        x = normed(self.norm2, None, ctx, h, branch)
        return h, ops.ScaledBranch(self.ffn.forward(ctx, x), self.scale2_f)


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """One norm whose output both branches read: h += mixer(n) + ffn(n), n = norm1(h).  The
    feed-forward branch may be absent (``LayerSpec.ffn`` None).  The sum of the two branches is
    formed in 32-bit (by a feed-forward with ``takes_addend``, in its last kernel) and returned still
    to be added; the norm that follows adds it to the stream."""

    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.ffn = FEED_FORWARDS.build(spec.ffn) if spec.ffn is not None else None
        if spec.extra:
            raise ValueError(f"the parallel arrangement has no parts {sorted(spec.extra)}")

    def children(self):
        n = self.names
        out = {n["norm1"]: self.norm1, n["mixer"]: self.mixer}
        if self.ffn is not None:
            out[n["ffn"]] = self.ffn
        return out

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        x = normed(self.norm1, None, ctx, h, delta)
        a = self.mixer.forward(ctx, x, cache)
        if self.ffn is None:
            return h, a
        if getattr(self.ffn, "takes_addend", False):
            return h, self.ffn.forward(ctx, x, addend=a)
        f = self.ffn.forward(ctx, x)
        both = torch.zeros((ctx.T, h.shape[1]), dtype=torch.float32, device=h.device)
        ops.stream_add(both, a)
        ops.stream_add(both, f)
        return h, both.view(1, ctx.T, h.shape[1])


def normed(norm, consumer, ctx: StepContext, h, delta):
    """h += delta; the normed rows for ``consumer``.  A norm that can and a
    consumer that takes it may pass the rows on unevaluated (ops.PendingNorm);
    a norm that does not know of pending products gets the product itself, and
    one that does not know of joining branches finds the branch joined."""
    if isinstance(delta, ops.JoiningBranch) and not getattr(norm, "joins_branches", False):
        delta = delta.join(h)
    if isinstance(delta, ops.ScaledBranch) and not getattr(norm, "takes_scaled", False):
        delta = delta.join(h)
    if getattr(norm, "can_defer", False):
        return norm.forward(ctx, h, delta, lazy=getattr(consumer, "takes_pending_norm", False))
    if isinstance(delta, ops.PendingLinear):
        delta = delta.run()
    return norm.forward(ctx, h, delta)


def stream_rows(ctx: StepContext, h, delta):
    """h += delta, and the stream's rows as a branch reads them when no norm stands in front of it:
    h itself in a 32-bit step, its copy in the step's type otherwise (a joining branch's kernel
    writes that copy on its way)."""
    if isinstance(delta, ops.JoiningBranch):
        if ctx.dtype == torch.float32:
            delta.join(h)
            return h
        out = torch.empty(h.shape, dtype=ctx.dtype, device=h.device)
        return ops.branch_join(h, delta.y, delta.weight, delta.mult, delta.eps, shift=delta.shift, out=out)
    if isinstance(delta, ops.ScaledBranch):
        delta = delta.join(h)
    if delta is not None:
        ops.stream_add(h, delta)
    return ops.cast(h, ctx.dtype)


@BLOCKS.register("normed_branches")
class NormedBranchesBlock(Block):
    """Every branch reads the residual stream itself and passes a norm on its way back:

        h += norm1(mixer(h));  h += norm2(ffn(h));  h += side_norm(side(h))

    The feed-forward branch may be absent (``LayerSpec.ffn`` None); the third branch is there when
    ``LayerSpec.extra`` has "side" (a feed-forward of the registry, one that may look at the step's
    token ids) and "side_norm" (its norm).  A branch joins in the kernel that prepares the next
    branch's input (ops.JoiningBranch); the block returns its last branch still to be joined."""

    def __init__(self, spec: LayerSpec):
        self.names = dict(spec.names)
        self.norm1 = NORMS.build(spec.norm1)
        self.mixer = MIXERS.build(spec.mixer)
        self.ffn = FEED_FORWARDS.build(spec.ffn) if spec.ffn is not None else None
        self.norm2 = NORMS.build(spec.norm2) if self.ffn is not None else None
        unknown = set(spec.extra) - {"side", "side_norm"}
        if unknown or (("side" in spec.extra) != ("side_norm" in spec.extra)):
            raise ValueError(f"the normed-branches arrangement takes 'side' with 'side_norm', not {sorted(spec.extra)}")
        self.side = FEED_FORWARDS.build(spec.extra["side"]) if "side" in spec.extra else None
        self.side_norm = NORMS.build(spec.extra["side_norm"]) if self.side is not None else None
        for norm in (self.norm1, self.norm2, self.side_norm):
            if norm is not None and not hasattr(norm, "branch"):
                raise ValueError(f"a branch's norm must be able to join it to the stream; {type(norm).__name__} cannot")

    def children(self):
        n = self.names
        out = {n["norm1"]: self.norm1, n["mixer"]: self.mixer}
        if self.ffn is not None:
            out.update({n["norm2"]: self.norm2, n["ffn"]: self.ffn})
        if self.side is not None:
            out.update({n["side"]: self.side, n["side_norm"]: self.side_norm})
        return out

    def forward(self, ctx: StepContext, h, delta, cache: LayerCache):
        x = stream_rows(ctx, h, delta)
        branch = self.norm1.branch(self.mixer.forward(ctx, x, cache))
        if self.ffn is not None:
            x = stream_rows(ctx, h, branch)
            branch = self.norm2.branch(self.ffn.forward(ctx, x))
        if self.side is not None:
            x = stream_rows(ctx, h, branch)
            branch = self.side_norm.branch(self.side.forward(ctx, x))
        return h, branch
