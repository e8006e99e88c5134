"""Two mixers side by side: both read the same input, and the layer's mixer
output is a weighted sum of theirs,

    y = left_scale * left(x) + right_scale * right(x),

formed in 32-bit.  The two are any mixers of the registry (``left``, ``right``:
PartSpecs); their tensors stand under ``left.`` and ``right.``.  The pair may
keep pages (one of the two: its ``cache_spec``), one state slot tensor (one of
the two: its ``state_spec``) and any further states of either, which reach the
child under its own names.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS
from ..config.specs import PartSpec
from ..kernels import ops
from .base import LayerCache, Mixer, StepContext


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    def __init__(self, left: PartSpec, right: PartSpec, left_scale: float = 1.0, right_scale: float = 1.0,
                 names: Optional[dict] = None):
        self.left, self.right = MIXERS.build(left), MIXERS.build(right)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        n = dict(left="left.", right="right.")
        n.update(names or {})
        self.names = n
        for what in ("cache_spec", "state_spec"):
            if getattr(self.left, what)() is not None and getattr(self.right, what)() is not None:
                raise ValueError(f"two mixers side by side: only one of them may have a {what}")
        self.graph_safe = self.left.graph_safe and self.right.graph_safe
        # a left mixer that can leave its output bias to us: the weighted sum's kernel adds it
        if hasattr(self.left, "defer_bias"):
            self.left.defer_bias = True

    def children(self):
        return {self.names["left"]: self.left, self.names["right"]: self.right}

    def cache_spec(self):
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self):
        return self.left.state_spec() or self.right.state_spec()

    def further_states(self):
        out = {"left." + k: v for k, v in self.left.further_states().items()}
        out.update({"right." + k: v for k, v in self.right.further_states().items()})
        return out

    def step_planner(self):
        # both children's planners are found by the runner's walk over the parts
        return None

    @staticmethod
    def _for_child(cache: LayerCache, side: str) -> LayerCache:
        prefix = "mixer." + side + "."
        states = {"mixer." + k[len(prefix):]: v for k, v in cache.states.items() if k.startswith(prefix)}
        return LayerCache(group=cache.group, pages=cache.pages, state=cache.state, writes=cache.writes, states=states)

    @staticmethod
    def _tensor(y):
        """What a mixer returned, as one tensor [T, H]."""
        if isinstance(y, ops.PendingLinear):
            y = y.run()
        return ops.sum_parts(y, torch.float32) if y.dim() == 3 else y

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        a = self._tensor(self.left.forward(ctx, x, self._for_child(cache, "left")))
        b = self._tensor(self.right.forward(ctx, x, self._for_child(cache, "right")))
        bias = getattr(self.left, "o_bias_f", None) if getattr(self.left, "defer_bias", False) else None
        return ops.weighted_sum(a, self.left_scale, b, self.right_scale, bias)
