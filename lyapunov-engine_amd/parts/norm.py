"""RMSNorm over the hidden dimension, fused with the residual add.

x * rsqrt(mean(x^2) + eps) * weight, all in 32-bit, as the reference's eager
path (python/lyapunov_engine/ops.py:49-50) and kernel
(csrc/kernels/fused_rmsnorm_swiglu.cu:83-84, 96-101).  The reference's model adds
the residual separately (models/llama.py:158, 164); here the add rides in the
norm that follows it, on a float residual stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import NORMS
from ..kernels import ops
from .base import Norm, StepContext, WeightSource, WeightSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, tensor: str = "weight", one_plus: bool = False):
        """``tensor``: what the weight is called after the part's prefix ("" where the prefix is
        the tensor's whole name).  ``one_plus``: the tensor is stored around zero and the norm
        multiplies by 1 + tensor (the sum is formed once, in 32-bit)."""
        self.size = size
        self.eps = float(eps)
        self.tensor = tensor
        self.one_plus = bool(one_plus)
        self.weight: Optional[torch.Tensor] = None
        self._weight_f: Optional[torch.Tensor] = None
        if self.one_plus:
            self.can_defer = False     # the folded forms take the stored tensor as the multiplier

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.size,)),), init="normal" if self.one_plus else "ones")]

    @property
    def weight_f(self) -> torch.Tensor:
        """The multipliers as float (made on first use; a norm's weights do not change)."""
        if self._weight_f is None:
            w = self.weight.float()
            self._weight_f = (1.0 + w if self.one_plus else w).contiguous()
        return self._weight_f

    def branch(self, y, mult: float = 1.0) -> "ops.JoiningBranch":
        """``y`` as a branch that joins the residual stream through this norm: mult * rmsnorm(y) * weight."""
        if isinstance(y, ops.PendingLinear):
            y = y.run()
        if y.dim() == 3:
            y = y[0] if y.shape[0] == 1 else ops.sum_parts(y, torch.float32)     # one slice: nothing to add up
        return ops.JoiningBranch(y, self.weight_f, self.eps, mult)

    # A delta may be an ops.JoiningBranch: the sum and this norm are then one kernel.
    joins_branches = True

    # With ``lazy`` the norm may add the delta and hand the rows on as an
    # ops.PendingNorm for the consumer's kernel to norm on its way in.
    can_defer = True

    def forward(self, ctx: StepContext, h, delta=None, rows=None, lazy=False, conv=None):
        """``conv``: see ``ops.branch_join``; the caller has checked that it applies (delta None or a
        joining branch, every row a request of one token, sizes that ``ops.branch_join_takes_conv``)."""
        if isinstance(delta, ops.JoiningBranch) or conv is not None:
            n = h.shape[0] if rows is None else rows.numel()
            out = torch.empty((n, self.size), dtype=ctx.dtype, device=h.device)
            if delta is None:
                return ops.branch_join(h, None, None, 1.0, 0.0, next_weight=self.weight_f, eps_next=self.eps, out=out,
                                       rows=rows, conv=conv)
            return ops.branch_join(h, delta.y, delta.weight, delta.mult, delta.eps, shift=delta.shift,
                                   next_weight=self.weight_f, eps_next=self.eps, out=out, rows=rows, conv=conv)
        if lazy and rows is None:
            pending, delta = ops.rmsnorm_pending(h, self.weight, self.eps, ctx.dtype, delta)
            if pending is not None:
                return pending
        n = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=ctx.dtype, device=h.device)
        return ops.rmsnorm(h, self.weight_f if self.one_plus else self.weight, self.eps, out, delta=delta, rows=rows)


@NORMS.register("group_rmsnorm")
class GroupRMSNorm(Norm):
    """RMS norm in groups: a row is cut into ``groups`` equal consecutive parts, each divided by its
    own sqrt(mean(part^2) + eps), and the whole row multiplied by the weight.  All in 32-bit.  The
    norm adds what is still to be added to the stream on its way: a tensor, float partial sums, or
    an ``ops.ScaledBranch`` (a branch times a learned vector), in the same kernel."""

    takes_scaled = True

    def __init__(self, size: int, eps: float, groups: int = 1, tensor: str = "weight"):
        if groups < 1 or size % groups:
            raise ValueError(f"rows of {size} values do not split into {groups} equal groups")
        self.size, self.eps, self.groups, self.tensor = int(size), float(eps), int(groups), tensor
        self.weight: Optional[torch.Tensor] = None
        self._weight_f: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.size,)),), init="ones")]

    @property
    def weight_f(self) -> torch.Tensor:
        if self._weight_f is None:
            self._weight_f = self.weight.float().contiguous()
        return self._weight_f

    def forward(self, ctx: StepContext, h, delta=None, rows=None, out_dtype=None):
        """``out_dtype``: the normed rows' type (None: the step's activations)."""
        scale = None
        if isinstance(delta, ops.ScaledBranch):
            delta, scale = delta.y, delta.scale
        if isinstance(delta, ops.PendingLinear):
            delta = delta.run()
        n = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.size), dtype=out_dtype or ctx.dtype, device=h.device)
        return ops.group_rmsnorm(h, self.weight_f, self.groups, self.eps, out, delta=delta, scale=scale, rows=rows)
