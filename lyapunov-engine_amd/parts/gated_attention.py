"""Grouped-query softmax attention assembled from options, for layers whose
projections are biased, normed or rotated in one of several ways, whose values
are their keys or are blended with an earlier layer's, whose scores are capped
or pay for distance, and whose heads pass a gate.

Per token x at position p, with H query heads and G key/value heads (query head
h reads key/value head h // (H / G)), keys and queries of ``dim`` values a head,
values of ``vdim``:

    q = W_q x (+ b_q),  k = W_k x (+ b_k),  v = W_v x (+ b_v)    one product with the gate's, 32-bit out
    values "keys": v = k as projected (there is no W_v; vdim = dim)
    value_mix "give": v (unblended, 32-bit) is left for later layers of the step;
              "take": v <- (1 - m) v + m v_given, m a learned number; what is blended is what the pages keep
    norm "head":  q, k <- x / rms(x) over every head (times a weight [dim] shared by the heads when ``norm_weight``)
         "whole": q, k <- x / rms(x) * w over the whole projection, all heads at once
    the first rotary_dim values of every head turn by p * f_i: pairs (2i, 2i + 1) ("neighbours") or (i, i + half) ("halves")
    s_j = scale * q_h . k_j;  cap > 0: s_j <- cap * tanh(s_j / cap);  slope_power > 0: s_j -= 2^(-slope_power (h + 1) / H) * (p - j)
    position p sees j <= p, and with a window only p - j < window
    weights = softmax over the visible keys; the denominator also holds exp(sink_h) ("learned") or 1 ("zero")
    gate "head": head h's output times sigmoid(W_g x)_h;  "element": every value times its own sigmoid(W_g x)
    y = W_o concat_h(...)

Keys and values go to the request's pages first (keys [kv head][slot][dim],
values [kv head][vdim][slot]) and attention reads pages only, so a whole prompt,
a portion and a decoded token take one path.  Heads with dim == vdim in
multiples of 16 (up to 256) run on the matrix-core kernels of
``parts.attention``; any other sizes on the row-by-row kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from .attention import AttentionWork, decode_launch, prefill_launch
from .base import LayerCache, Mixer, PagedSpec, StepContext, WeightSource, WeightSpec

_WORK = AttentionWork()

NORMS_OF_QK = ("none", "head", "whole")
PAIRINGS = ("neighbours", "halves")
SINKS = ("none", "learned", "zero")
GATES = ("none", "head", "element")
VALUE_MIXES = ("none", "give", "take")


@MIXERS.register("gated_attention")
class GatedAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int = 0, bias: bool = False, norm: str = "none", norm_weight: bool = True, eps: float = 1e-6,
                 position: Optional[PartSpec] = None, pairing: str = "neighbours", values: str = "own",
                 value_mix: str = "none", value_mix_key: str = "values", cap: float = 0.0, slope_power: float = 0.0,
                 sink: str = "none", gate: str = "none", names: Optional[dict] = None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not split over {num_kv_heads} key/value heads")
        if dim <= 0 or vdim <= 0 or window < 0 or cap < 0 or slope_power < 0:
            raise ValueError(f"attention: heads of {dim}/{vdim}, window {window}, cap {cap}, slope power {slope_power}")
        for what, value, known in (("norm", norm, NORMS_OF_QK), ("pairing", pairing, PAIRINGS), ("sink", sink, SINKS),
                                   ("gate", gate, GATES), ("value_mix", value_mix, VALUE_MIXES), ("values", values, ("own", "keys"))):
            if value not in known:
                raise ValueError(f"attention: {what} {value!r}; known: {list(known)}")
        if values == "keys" and vdim != dim:
            raise ValueError(f"values that are the keys have the keys' size, {dim}, not {vdim}")
        if norm == "whole" and not norm_weight:
            raise ValueError("a norm over the whole projection comes with its weights")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.scale, self.window = int(dim), int(vdim), float(scale), int(window)
        self.has_bias, self.norm, self.norm_weight, self.eps = bool(bias), norm, bool(norm_weight) and norm != "none", float(eps)
        self.position = POSITION_ENCODINGS.build(position) if position is not None else None
        if self.position is not None and self.position.rotary_dim > dim:
            raise ValueError("more rotated dimensions than a head has")
        self.pairing, self.values_from_keys = pairing, values == "keys"
        self.value_mix, self.value_mix_key = value_mix, "value_mix:" + value_mix_key
        self.cap, self.slope_power, self.sink_kind, self.gate = float(cap), float(slope_power), sink, gate
        n = dict(q="q", k="k", v="v", bias=".b", q_norm="q.norm", k_norm="k.norm", mix="vmix", sink="sink", g="g", o="o")
        n.update(names or {})
        self.names = n
        self.matrix_cores = self.dim == self.vdim and self.dim % 16 == 0 and self.dim <= 256
        self.gate_cols = {"none": 0, "head": self.num_heads, "element": self.num_heads * self.vdim}[gate]
        self.in_proj = self.in_bias = self.o_proj = self.q_norm = self.k_norm = self.mix = self.sink = None
        self.in_bias_f = self.q_norm_f = self.k_norm_f = self.mix_f = self.sink_f = self.slopes_f = None

    def _projections(self) -> list:
        n, H, G = self.names, self.num_heads, self.num_kv_heads
        return [(n["q"], H * self.dim), (n["k"], G * self.dim)] + ([] if self.values_from_keys else [(n["v"], G * self.vdim)])

    def weight_specs(self):
        n, H, G, C = self.names, self.num_heads, self.num_kv_heads, self.hidden_size
        sizes = self._projections()
        specs = [WeightSpec("in_proj", tuple(WeightSource(name, (rows, C)) for name, rows in
                                             sizes + ([(n["g"], self.gate_cols)] if self.gate_cols else []))),
                 WeightSpec("o_proj", (WeightSource(n["o"], (C, H * self.vdim)),))]
        if self.has_bias:
            specs.append(WeightSpec("in_bias", tuple(WeightSource(name + n["bias"], (rows,)) for name, rows in sizes)))
        if self.norm_weight:
            nq, nk = (H * self.dim, G * self.dim) if self.norm == "whole" else (self.dim, self.dim)
            specs += [WeightSpec("q_norm", (WeightSource(n["q_norm"], (nq,)),), init="ones"),
                      WeightSpec("k_norm", (WeightSource(n["k_norm"], (nk,)),), init="ones")]
        if self.value_mix == "take":
            specs.append(WeightSpec("mix", (WeightSource(n["mix"], ()),)))
        if self.sink_kind == "learned":
            specs.append(WeightSpec("sink", (WeightSource(n["sink"], (H,)),)))
        return specs

    def children(self):
        return {"rotary.": self.position} if self.position is not None else {}

    def materialize(self, device, dtype):
        super().materialize(device, dtype)
        H = self.num_heads
        if self.has_bias:
            self.in_bias_f = self.in_bias.float().contiguous()
        if self.norm_weight:
            self.q_norm_f, self.k_norm_f = self.q_norm.float().contiguous(), self.k_norm.float().contiguous()
        if self.value_mix == "take":
            self.mix_f = self.mix.float().reshape(1).contiguous()
        if self.sink_kind == "learned":
            self.sink_f = self.sink.float().contiguous()
        elif self.sink_kind == "zero":
            self.sink_f = torch.zeros(H, dtype=torch.float32, device=device)
        if self.slope_power > 0:
            self.slopes_f = torch.tensor([2.0 ** (-self.slope_power * (h + 1) / H) for h in range(H)],
                                         dtype=torch.float64).float().to(device)

    def cache_spec(self):
        return PagedSpec.keys_and_values(self.num_kv_heads, self.dim, self.window, value_dim=self.vdim)

    def step_planner(self):
        return _WORK if self.matrix_cores else None

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        if not cache.writes:
            raise RuntimeError("this attention keeps its own keys and values")
        g, H, G = cache.group, self.num_heads, self.num_kv_heads
        pre = ops.linear(x, self.in_proj, out_dtype=torch.float32)
        other = None
        if self.value_mix == "take":
            other = ctx.workspace.get(self.value_mix_key)
            if other is None or other.shape[0] != ctx.T:
                raise RuntimeError("values to blend with: no earlier layer of this step has left any")
        q, kept = ops.qkv_prepare(
            pre, ctx.dtype, num_heads=H, num_kv_heads=G, dim=self.dim, vdim=self.vdim, slots=g.slot_mapping,
            kpool=cache.k, vpool=cache.v, page_size=g.page_size, bias=self.in_bias_f, norm=self.norm,
            q_weight=self.q_norm_f, k_weight=self.k_norm_f, eps=self.eps, positions=ctx.positions,
            table=self.position.table if self.position is not None else None, pairing=self.pairing,
            values_from_keys=self.values_from_keys, blend=self.mix_f if other is not None else None, other_values=other,
            keep_values=self.value_mix == "give")
        if kept is not None:
            ctx.workspace[self.value_mix_key] = kept
        make = torch.zeros if ctx.fixed is not None and ctx.fixed.tokens else torch.empty
        out = make((ctx.T, H * self.vdim), dtype=ctx.dtype, device=q.device)
        if not self.matrix_cores:
            ops.attn_rows(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.positions, ctx.ctx_len,
                          num_heads=H, num_kv_heads=G, dim=self.dim, vdim=self.vdim, scale=self.scale,
                          window=self.window, sink=self.sink_f, cap=self.cap, slopes=self.slopes_f)
        else:
            common = dict(num_heads=H, num_kv_heads=G, head_dim=self.dim, window=self.window, scale=self.scale,
                          sink=self.sink_f, cap=self.cap, slopes=self.slopes_f)
            sizes = dict(num_heads=H, num_kv_heads=G, head_dim=self.dim)
            work = ctx.plans[AttentionWork.key]
            pl = prefill_launch(work.meta, ctx.dtype, g.page_size, window=self.window, **sizes)
            if pl is not None:
                part_o = part_ml = None
                if pl["parts"] > 1:
                    part_o = ctx.scratch("attn_part_o", pl["part_o"])
                    part_ml = ctx.scratch("attn_part_ml", pl["part_ml"])
                ops.attn_prefill(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                                 work.arrays["tile_seq"], work.arrays["tile_q0"], pl["n_tiles"], pair=pl["pair"],
                                 parts=pl["parts"], part_o=part_o, part_ml=part_ml, **common)
            dec = decode_launch(work.meta, **sizes)
            if dec is not None:
                part_o = ctx.scratch("attn_part_o", dec["part_o"])
                part_ml = ctx.scratch("attn_part_ml", dec["part_ml"])
                ops.attn_decode(q, out, cache.k, cache.v, g.block_tables, ctx.q_start, ctx.ctx_len,
                                work.arrays.get("dec"), dec["n_dec"], part_o, part_ml, dec["max_parts"],
                                dec["part_keys"], **common)
        if self.gate_cols:
            at = pre.shape[1] - self.gate_cols
            ops.gate_mul(out, pre[:, at:], "sigmoid", per=self.vdim if self.gate == "head" else 1)
        return ops.linear(out, self.o_proj, out_dtype=ctx.dtype)
