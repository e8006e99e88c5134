"""Filters over time on what a branch reads.

"short_conv": a causal convolution with a few taps per channel, added to its
input: out_t = x_t + sum_j w[:, j] * x_(t - taps + 1 + j), with zeros before the
first token of a request.  The last taps - 1 inputs of every live request stay
in a state slot, so that a prompt may be cut anywhere and a decoded token sees
the tokens before it.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import FILTERS
from ..kernels import ops
from .base import InputFilter, StateSpec, StepContext, WeightSource, WeightSpec


@FILTERS.register("short_conv")
class CausalShortConv(InputFilter):
    def __init__(self, channels: int, taps: int, residual: bool = True, tensor: str = "weight"):
        if taps < 1:
            raise ValueError(f"a convolution needs at least one tap, not {taps}")
        self.channels, self.taps, self.residual, self.tensor = int(channels), int(taps), bool(residual), tensor
        self.weight: Optional[torch.Tensor] = None
        self.weight_f: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.channels, self.taps)),))]

    def materialize(self, device, dtype):
        self.weight_f = self.weight.float().contiguous()

    def state_spec(self):
        # the inputs are activations; they are kept as they were read
        return StateSpec((self.taps - 1, self.channels), None) if self.taps > 1 else None

    def fused(self, ctx: StepContext, state: Optional[torch.Tensor], width: int):
        """What ``ops.branch_join`` needs to run this filter behind a norm in one kernel (a step
        in which every request brings one token), or None where it cannot."""
        if not self.residual or width != self.channels or not ops.branch_join_takes_conv(width):
            return None
        return (self.weight_f, state, ctx.state_slots, ctx.positions)

    def forward(self, ctx: StepContext, x: torch.Tensor, state: Optional[torch.Tensor]) -> torch.Tensor:
        out = torch.empty_like(x)
        return ops.short_conv(x, self.weight_f, state, ctx.q_start, ctx.positions, ctx.state_slots, out, ctx.B,
                              residual=self.residual)


@FILTERS.register("token_shift")
class TokenShift(CausalShortConv):
    """Every channel moves a learned part of the way towards the previous token's value:
    out_t = x_t + (x_(t-1) - x_t) * mu, with x_(-1) = 0.  That is a convolution of two taps,
    (mu, 1 - mu), without the residual; the previous token's input is the state."""

    def __init__(self, channels: int, tensor: str = "weight"):
        super().__init__(channels, taps=2, residual=False, tensor=tensor)
        self.mix: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("mix", (WeightSource(self.tensor, (self.channels,)),))]

    def materialize(self, device, dtype):
        mu = self.mix.float()
        self.weight_f = torch.stack([mu, 1.0 - mu], dim=1).contiguous()

    def fused(self, ctx, state, width):
        return None
