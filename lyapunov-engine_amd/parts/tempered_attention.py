"""Grouped-query softmax attention with biased projections, a query multiplier
that grows with the position, and a sigmoid gate on the heads' outputs.

Per token x at position p, with H query heads and G key/value heads (query head
h reads key/value head h // (H / G)), keys and queries of ``dim`` values a head,
values of ``vdim``:

    q = W_q x + b_q,  k = W_k x + b_k,  v = W_v x + b_v      one product with the gate's, in 32-bit out
    q <- q * (1 + coef * ln(floor((p + 1) / every) + 1))     positions enter nowhere else
    weights = softmax over j <= p of scale * q_h . k_j
    y = W_o (concat_h(sum_j weights_j v_j) * sigmoid(W_g x)) + b_o

Keys and values go to the request's pages (keys [kv head][slot][dim], values
[kv head][vdim][slot]) and attention reads pages only, so a whole prompt, a
portion and a decoded token take one path.  Heads with dim == vdim in multiples
of 16 (up to 256) run on the matrix-core kernels of ``parts.attention``; any
other sizes on the row-by-row kernel.  The result is float (the output
projection's accumulators plus its bias).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS
from ..kernels import ops
from .attention import AttentionWork, decode_launch, prefill_launch
from .base import LayerCache, Mixer, PagedSpec, StepContext, WeightSource, WeightSpec

_WORK = AttentionWork()


@MIXERS.register("tempered_attention")
class TemperedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 temper_coef: float = 0.0, temper_every: int = 1, bias: bool = True, gate: bool = True,
                 names: Optional[dict] = None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not split over {num_kv_heads} key/value heads")
        if dim <= 0 or vdim <= 0 or temper_every < 1:
            raise ValueError(f"attention: heads of {dim}/{vdim}, a query multiplier every {temper_every} positions")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale = int(dim), int(vdim), float(scale)
        self.temper_coef, self.temper_every = float(temper_coef), int(temper_every)
        self.has_bias, self.has_gate = bool(bias), bool(gate)
        n = dict(q="q", k="k", v="v", g="g", o="o", bias=".b")
        n.update(names or {})
        self.names = n
        self.matrix_cores = self.dim == self.vdim and self.dim % 16 == 0 and self.dim <= 256
        self.in_proj = self.in_bias = self.o_proj = self.o_bias = None
        self.in_bias_f = self.o_bias_f = None
        # True: ``forward`` leaves the output projection's bias to its caller (``o_bias_f``), who adds it in a kernel of its own
        self.defer_bias = False

    def weight_specs(self):
        n, H, G, C = self.names, self.num_heads, self.num_kv_heads, self.hidden_size
        sizes = [(n["q"], H * self.dim), (n["k"], G * self.dim), (n["v"], G * self.vdim)]
        specs = [WeightSpec("in_proj", tuple(WeightSource(name, (rows, C)) for name, rows in
                                             sizes + ([(n["g"], H * self.vdim)] if self.has_gate else []))),
                 WeightSpec("o_proj", (WeightSource(n["o"], (C, H * self.vdim)),))]
        if self.has_bias:
            specs += [WeightSpec("in_bias", tuple(WeightSource(name + n["bias"], (rows,)) for name, rows in sizes)),
                      WeightSpec("o_bias", (WeightSource(n["o"] + n["bias"], (C,)),))]
        return specs

    def materialize(self, device, dtype):
        if self.has_bias:
            self.in_bias_f = self.in_bias.float().contiguous()
            self.o_bias_f = self.o_bias.float().contiguous()

    def cache_spec(self):
        return PagedSpec.keys_and_values(self.num_kv_heads, self.dim, 0, value_dim=self.vdim)

    def step_planner(self):
        return _WORK if self.matrix_cores else None

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        if not cache.writes:
            raise RuntimeError("this attention keeps its own keys and values")
        g, H, G = cache.group, self.num_heads, self.num_kv_heads
        pre = ops.linear(x, self.in_proj, out_dtype=torch.float32)
        q = ops.qkv_bias_temper_kv(pre, self.in_bias_f, ctx.positions, self.temper_coef, self.temper_every,
                                   g.slot_mapping, cache.k, cache.v, ctx.dtype, num_heads=H, num_kv_heads=G,
                                   dim=self.dim, vdim=self.vdim, page_size=g.page_size)
        make = torch.zeros if ctx.fixed is not None and ctx.fixed.tokens else torch.empty
        out = make((ctx.T, H * self.vdim), dtype=ctx.dtype, device=q.device)
        if not self.matrix_cores:
            ops.attn_rows(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.positions, ctx.ctx_len,
                          num_heads=H, num_kv_heads=G, dim=self.dim, vdim=self.vdim, scale=self.scale)
        else:
            common = dict(num_heads=H, num_kv_heads=G, head_dim=self.dim, window=0, scale=self.scale)
            work = ctx.plans[AttentionWork.key]
            pl = prefill_launch(work.meta, ctx.dtype, g.page_size, **{k: common[k] for k in ("num_heads", "num_kv_heads", "head_dim")})
            if pl is not None:
                part_o = part_ml = None
                if pl["parts"] > 1:
                    part_o = ctx.scratch("attn_part_o", pl["part_o"])
                    part_ml = ctx.scratch("attn_part_ml", pl["part_ml"])
                ops.attn_prefill(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                                 work.arrays["tile_seq"], work.arrays["tile_q0"], pl["n_tiles"], pair=pl["pair"],
                                 parts=pl["parts"], part_o=part_o, part_ml=part_ml, **common)
            dec = decode_launch(work.meta, **{k: common[k] for k in ("num_heads", "num_kv_heads", "head_dim")})
            if dec is not None:
                part_o = ctx.scratch("attn_part_o", dec["part_o"])
                part_ml = ctx.scratch("attn_part_ml", dec["part_ml"])
                ops.attn_decode(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                                work.arrays.get("dec"), dec["n_dec"], part_o, part_ml, dec["max_parts"],
                                dec["part_keys"], **common)
        if self.has_gate:
            at = (H + G) * self.dim + G * self.vdim
            ops.gate_mul(out, pre[:, at:at + H * self.vdim], "sigmoid")
        y = ops.linear(out, self.o_proj, out_dtype=torch.float32)
        if self.o_bias_f is not None and not self.defer_bias:
            ops.add_row(y, self.o_bias_f)
        return y
