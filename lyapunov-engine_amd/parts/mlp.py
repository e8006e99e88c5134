"""SiLU-gated feed-forward.

down( silu(gate(x)) * up(x) ), no biases, with gate and up as one matrix whose
first rows are the gate (python/lyapunov_engine/models/llama.py:109-122;
models/weight_loader.py:155-163 builds cat([gate, up], dim=0); the activation is
python/lyapunov_engine/ops.py:72-73).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import FEED_FORWARDS
from ..kernels import ops
from .base import FeedForward, StepContext, WeightSource, WeightSpec


@FEED_FORWARDS.register("dense")
class DenseFeedForward(FeedForward):
    """down(act(up(x))), no gate and no biases.  ``activation``: "xielu", with its two learned
    numbers p, q in one tensor (z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (e^z - 1 - z)
    + z/2), or "gelu_tanh"."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "xielu",
                 names: Optional[dict] = None):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {sorted(ops.ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = int(hidden_size), int(intermediate_size), activation
        n = dict(up="up", down="down", act="act")
        n.update(names or {})
        self.names = n
        self.up_proj: Optional[torch.Tensor] = None
        self.down_proj: Optional[torch.Tensor] = None
        self.act_params: Optional[torch.Tensor] = None
        self.act_params_f: Optional[torch.Tensor] = None

    def weight_specs(self):
        n = self.names
        specs = [WeightSpec("up_proj", (WeightSource(n["up"], (self.intermediate_size, self.hidden_size)),)),
                 WeightSpec("down_proj", (WeightSource(n["down"], (self.hidden_size, self.intermediate_size)),))]
        if self.activation == "xielu":
            specs.append(WeightSpec("act_params", (WeightSource(n["act"], (2,)),)))
        return specs

    def materialize(self, device, dtype):
        if self.act_params is not None:
            self.act_params_f = self.act_params.float().contiguous()

    def forward(self, ctx: StepContext, x):
        up = ops.linear(x, self.up_proj, out_dtype=ctx.dtype)
        ops.activation(up, self.activation, self.act_params_f)
        return ops.linear(up, self.down_proj, out_dtype=ctx.dtype)


@FEED_FORWARDS.register("gated_dense")
class GatedDense(FeedForward):
    """down(act(gate(x)) * up(x)), no biases; ``activation``: "silu" or "gelu_tanh" (the tanh form of
    gelu).  Gate and up are one matrix whose first rows are the gate."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", names: Optional[dict] = None):
        if activation not in ops.GLU_ACTIVATIONS:
            raise ValueError(f"unknown gate activation {activation!r}; known: {sorted(ops.GLU_ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size, self.activation = int(hidden_size), int(intermediate_size), activation
        n = dict(gate="gate", up="up", down="down")
        n.update(names or {})
        self.names = n
        self.gate_up_proj: Optional[torch.Tensor] = None
        self.down_proj: Optional[torch.Tensor] = None

    def weight_specs(self):
        n, shape = self.names, (self.intermediate_size, self.hidden_size)
        return [WeightSpec("gate_up_proj", (WeightSource(n["gate"], shape), WeightSource(n["up"], shape))),
                WeightSpec("down_proj", (WeightSource(n["down"], (self.hidden_size, self.intermediate_size)),))]

    def forward(self, ctx: StepContext, x):
        act = ops.glu_act(ops.linear(x, self.gate_up_proj, out_dtype=ctx.dtype), self.activation)
        return ops.linear(act, self.down_proj, out_dtype=ctx.dtype)


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        # Rows of the fused matrix in tiles of 16 (eight gates, their eight ups) let a
        # decode step gate inside the product; widths that are no multiple of 8 keep
        # the plain order, gates first.
        self.interleave = 8 if intermediate_size % 8 == 0 else 0
        self.gate_up_proj: Optional[torch.Tensor] = None
        self.down_proj: Optional[torch.Tensor] = None

    def weight_specs(self):
        shape = (self.intermediate_size, self.hidden_size)
        return [
            WeightSpec("gate_up_proj", (WeightSource("gate_proj.weight", shape), WeightSource("up_proj.weight", shape)),
                       interleave=self.interleave),
            WeightSpec("down_proj", (WeightSource("down_proj.weight", (self.hidden_size, self.intermediate_size)),)),
        ]

    takes_pending_norm = True   # x may be an ops.PendingNorm: the gate/up product norms on its way in

    def forward(self, ctx: StepContext, x):
        act = ops.linear_swiglu(x, self.gate_up_proj, self.interleave)
        return ops.linear(act, self.down_proj, out_dtype=ctx.dtype, may_split=True, pending=True)


@FEED_FORWARDS.register("token_gated")
class TokenGatedProjection(FeedForward):
    """A small branch that the token itself gates: with e the token's row of a table (``dim``
    values; the table may be a column range of a wider tensor that several layers share),

        y = W_proj (gelu_tanh(W_gate x) * e)

    ``table``: the tensor's whole name in the files; ``table_width`` its columns, of which this part
    takes ``dim`` from ``column`` on."""

    def __init__(self, hidden_size: int, dim: int, vocab_size: int, table: str, table_width: Optional[int] = None,
                 column: int = 0, names: Optional[dict] = None):
        width = dim if table_width is None else int(table_width)
        if dim <= 0 or vocab_size <= 0 or not 0 <= column <= width - dim:
            raise ValueError(f"token-gated branch: {dim} values from column {column} of a table of {width}")
        self.hidden_size, self.dim, self.vocab_size = int(hidden_size), int(dim), int(vocab_size)
        self.table_name, self.table_width, self.column = table, width, int(column)
        n = dict(gate="gate", proj="proj")
        n.update(names or {})
        self.names = n
        self.gate_proj: Optional[torch.Tensor] = None
        self.out_proj: Optional[torch.Tensor] = None
        self.table: Optional[torch.Tensor] = None

    def weight_specs(self):
        n = self.names
        return [WeightSpec("gate_proj", (WeightSource(n["gate"], (self.dim, self.hidden_size)),)),
                WeightSpec("out_proj", (WeightSource(n["proj"], (self.hidden_size, self.dim)),)),
                WeightSpec("table", (WeightSource(self.table_name, (self.vocab_size, self.table_width), absolute=True,
                                                  columns=(self.column, self.column + self.dim)),))]

    def forward(self, ctx: StepContext, x):
        p = ops.linear(x, self.gate_proj, out_dtype=torch.float32)
        g = ops.gather_gelu_mul(p, ctx.token_ids, self.table)
        return ops.linear(g, self.out_proj, out_dtype=ctx.dtype)
