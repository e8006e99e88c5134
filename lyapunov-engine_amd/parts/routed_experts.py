"""A feed-forward that routes every token to a few of many small experts.

    z = W_r x + b                       router logits, in 32-bit
    the ``top`` experts with the largest z; their weights: the softmax over those z alone
    expert e:  g = min(W_gate,e x, limit), u = clamp(W_up,e x, -limit, limit)
               y_e = W_down,e (g * sigmoid(gate_slope * g) * (u + 1))
    out = sum over the chosen e of weight_e * y_e   (+ a shared expert of the same form, run for every token)

No biases in the experts.  On the device nothing is counted on the host: the
(token, choice) pairs are sorted by expert in one kernel, the two products walk
a list of row tiles that kernel leaves (grids sized for the most tiles there can
be), and the last kernel adds a token's weighted expert outputs, the shared
expert's and, when the layer's arrangement hands it one, the other branch's
output in 32-bit.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..kernels import ops
from .base import FeedForward, StepContext, WeightSource, WeightSpec


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    # ``forward`` takes the other branch's output as ``addend`` and returns the sum of both.
    takes_addend = True
    # A list here receives every call's chosen experts (int32 [T, top], on the device), in the order
    # of the calls: for load statistics, and for comparing a run with another that must route alike.
    choices_log: Optional[list] = None

    def __init__(self, hidden_size: int, num_experts: int, top: int, intermediate_size: int, limit: float,
                 gate_slope: float = 1.702, shared_size: int = 0, shared_limit: float = 0.0,
                 names: Optional[dict] = None):
        if not 1 <= top <= num_experts or intermediate_size <= 0 or shared_size < 0:
            raise ValueError(f"routed experts: {top} of {num_experts} experts of {intermediate_size}, shared {shared_size}")
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.intermediate_size, self.limit, self.gate_slope = int(intermediate_size), float(limit), float(gate_slope)
        self.shared_size, self.shared_limit = int(shared_size), float(shared_limit)
        n = dict(router="router", router_bias="router.b", expert="e{j}.", shared="shared.", gate="gate", up="up",
                 down="down")
        n.update(names or {})
        self.names = n
        # A shared expert of the routed experts' size and limit is kept as one more matrix behind
        # theirs and rides in their products as an expert every token uses with weight 1.
        self.shared_folded = self.shared_size == self.intermediate_size and self.shared_limit == self.limit
        self.router = self.router_bias = self.gate_up = self.down = self.shared_gate_up = self.shared_down = None
        self.router_f = self.router_bias_f = None

    def weight_specs(self):
        n, E, I, H = self.names, self.num_experts, self.intermediate_size, self.hidden_size
        gate_up, down = [], []
        for j in range(E):
            e = n["expert"].format(j=j)
            gate_up += [WeightSource(e + n["gate"], (I, H)), WeightSource(e + n["up"], (I, H))]
            down.append(WeightSource(e + n["down"], (H, I)))
        if self.shared_folded:
            s = n["shared"]
            gate_up += [WeightSource(s + n["gate"], (I, H)), WeightSource(s + n["up"], (I, H))]
            down.append(WeightSource(s + n["down"], (H, I)))
        specs = [WeightSpec("router", (WeightSource(n["router"], (E, H)),)),
                 WeightSpec("router_bias", (WeightSource(n["router_bias"], (E,)),)),
                 WeightSpec("gate_up", tuple(gate_up)), WeightSpec("down", tuple(down))]
        if self.shared_size and not self.shared_folded:
            s, S = n["shared"], self.shared_size
            specs += [WeightSpec("shared_gate_up", (WeightSource(s + n["gate"], (S, H)), WeightSource(s + n["up"], (S, H)))),
                      WeightSpec("shared_down", (WeightSource(s + n["down"], (H, S)),))]
        return specs

    def materialize(self, device, dtype):
        E, I, H = self.num_experts, self.intermediate_size, self.hidden_size
        # the router works in 32-bit whatever the activations are
        self.router_f = self.router.float().contiguous()
        self.router_bias_f = self.router_bias.float().contiguous()
        self.router = None
        stacked = E + (1 if self.shared_folded else 0)
        self.gate_up = self.gate_up.view(stacked, 2 * I, H)      # per expert: gate rows, then up rows
        self.down = self.down.view(stacked, H, I)

    def forward(self, ctx: StepContext, x, addend=None):
        """-> float [1, T, hidden] (one slice of partial sums): the experts' weighted outputs, the
        shared expert's and ``addend`` (the other branch's output, activations [T, hidden])."""
        T = x.shape[0]
        always = self.num_experts if self.shared_folded else -1
        idx, wgt, plan = ops.moe_route_from(x, self.router_f, self.router_bias_f, self.top, always,
                                            sort_for=self.gate_up.shape[0])
        if RoutedExperts.choices_log is not None:
            RoutedExperts.choices_log.append(idx[:, :self.top])
        act = ops.moe_gemm(x, self.gate_up, plan, gated=True, limit=self.limit, alpha=self.gate_slope)
        y = ops.moe_gemm(act, self.down, plan, gated=False)
        shared = None
        if self.shared_size and not self.shared_folded:
            gu = ops.linear(x, self.shared_gate_up, out_dtype=ctx.dtype)
            shared = ops.linear(ops.glu_clamped(gu, self.shared_limit, self.gate_slope), self.shared_down,
                                out_dtype=ctx.dtype)
        if addend is not None:
            addend = ops.as_delta(addend, ctx.dtype)
        return ops.moe_combine(y, plan, wgt, T, addend=addend, shared=shared)


@FEED_FORWARDS.register("group_routed_experts")
class GroupRoutedExperts(FeedForward):
    """Experts chosen by sigmoid scores within the best groups:

        s = sigmoid(W_r x)                                 in 32-bit
        choice scores c = s + correction; the experts form ``groups`` equal groups of neighbours, a
        group's score is the sum of its two largest c, and only experts of the ``keep`` best groups
        can be chosen; the ``top`` largest c among those are
        weights: the chosen experts' s over their sum (+ 1e-20), times ``scale``
        expert e:  y_e = W_down,e relu(W_up,e x)^2         no gate, no biases
        out = sum over the chosen e of weight_e * y_e

    The (token, choice) pairs are sorted by expert on the device; both products walk the sorted
    tiles (``ops.moe_gemm``: the first gathers its rows by token and squares the positive part of
    its result), the last kernel adds a token's weighted outputs in 32-bit."""

    choices_log: Optional[list] = None   # as RoutedExperts.choices_log

    def __init__(self, hidden_size: int, num_experts: int, top: int, intermediate_size: int, groups: int = 1,
                 keep: int = 1, scale: float = 1.0, names: Optional[dict] = None):
        if not 1 <= top <= num_experts or intermediate_size <= 0:
            raise ValueError(f"routed experts: {top} of {num_experts} experts of {intermediate_size}")
        if groups < 1 or num_experts % groups or not 1 <= keep <= groups or keep * (num_experts // groups) < top:
            raise ValueError(f"routed experts: {num_experts} experts in {groups} groups of which {keep} are kept "
                             f"cannot give {top} choices")
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.intermediate_size, self.groups, self.keep, self.scale = int(intermediate_size), int(groups), int(keep), float(scale)
        n = dict(router="router", correction="correction", expert="e{j}.", up="up", down="down")
        n.update(names or {})
        self.names = n
        self.router = self.correction = self.up = self.down = None
        self.router_f = self.correction_f = None

    def weight_specs(self):
        n, E, I, H = self.names, self.num_experts, self.intermediate_size, self.hidden_size
        ups = tuple(WeightSource(n["expert"].format(j=j) + n["up"], (I, H)) for j in range(E))
        downs = tuple(WeightSource(n["expert"].format(j=j) + n["down"], (H, I)) for j in range(E))
        return [WeightSpec("router", (WeightSource(n["router"], (E, H)),)),
                WeightSpec("correction", (WeightSource(n["correction"], (E,)),)),
                WeightSpec("up", ups), WeightSpec("down", downs)]

    def materialize(self, device, dtype):
        E, I, H = self.num_experts, self.intermediate_size, self.hidden_size
        self.router_f = self.router.float().contiguous()
        self.correction_f = self.correction.float().contiguous()
        self.router = None
        self.up = self.up.view(E, I, H)
        self.down = self.down.view(E, H, I)

    def forward(self, ctx: StepContext, x):
        """-> float [1, T, hidden] (one slice of partial sums)."""
        idx, wgt = ops.moe_route_grouped(x, self.router_f, self.correction_f, self.top, self.groups, self.keep, self.scale)
        if GroupRoutedExperts.choices_log is not None:
            GroupRoutedExperts.choices_log.append(idx)
        plan = ops.moe_sort(idx, self.num_experts)
        act = ops.moe_gemm(x, self.up, plan, gated=False, gather=True, relu2=True)
        y = ops.moe_gemm(act, self.down, plan, gated=False)
        return ops.moe_combine(y, plan, wgt, x.shape[0])
