"""Mixers that carry a matrix per head instead of keys: a gated delta rule and
gated linear attention, both with a decay per head and key channel; a time mix
whose output gives the current token a bonus ("time_mix"), and a state-space
layer whose decay per head follows a step size ("selective_state_space"), both
described at their classes.

Per head, with S a matrix [dim x vdim] that starts at zero and lives in 32-bit
in a state slot of the request:

  "gated_delta_rule"
    q, k (G heads of dim), v (H heads of vdim): projections, each through a short causal
    convolution per channel and silu; q and k made unit vectors per head, q times dim^(-1/2);
    query head h reads q/k head h // (H / G)
    g = exp(-exp(A_h) * softplus(W_a2 (W_a1 x) + b_dt))      one decay per head and key channel
    beta = sigmoid(W_b x)                                    one per head
    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    y = W_o concat_h( o_h / rms(o_h) * w * sigmoid(W_g2 (W_g1 x)) )

  "gated_linear_attention"
    q = W_q x * dim^(-1/2), k = W_k x (H heads of dim), v = W_v x (H heads of vdim)
    a = sigmoid(W_a2 (W_a1 x) + b)^(1 / tau)                 one decay per head and key channel
    S <- diag(a) S + k v^T;  o = S^T q
    y = W_o concat_h( o_h / rms(o_h) * w * silu(W_g x) )

Everything that reads x is one product; the inner sizes of the low-rank pairs
(W_a1, W_g1) are whatever the file's tensors have.  Decays, unit vectors, beta,
the recurrence and the heads' norm are 32-bit (``ops.linear_scan``,
``ops.head_norm_gate``); the state is kept transposed, [heads, vdim, dim].
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import MIXERS
from ..kernels import ops
from .base import LayerCache, Mixer, StateSpec, StepContext, WeightSource, WeightSpec, free_size

MADE_UP_RANK = 16   # inner size of the low-rank pairs when weights are made up


def _scan_out(ctx: StepContext, width: int) -> torch.Tensor:
    """The recurrence's float output; zeroed where a recorded prompt step has rows that belong to no request."""
    make = torch.zeros if ctx.fixed is not None and ctx.fixed.tokens else torch.empty
    return make((ctx.T, width), dtype=torch.float32, device=ctx.device)


@MIXERS.register("gated_delta_rule")
class GatedDeltaRule(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, conv_taps: int,
                 eps: float, names: Optional[dict] = None):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not split over {num_kv_heads} query/key heads")
        if not 0 < dim <= ops.LINEAR_SCAN_MAX_DIM or vdim <= 0 or conv_taps < 1:
            raise ValueError(f"gated delta rule: heads of {dim}/{vdim} (keys of up to {ops.LINEAR_SCAN_MAX_DIM}), "
                             f"{conv_taps} taps")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.taps, self.eps = int(dim), int(vdim), int(conv_taps), float(eps)
        n = dict(q="q", k="k", v="v", q_conv="q.conv", k_conv="k.conv", v_conv="v.conv", beta="b", decay_log="A_log",
                 decay_in="a1", decay_out="a2", decay_bias="dt_bias", gate_in="g1", gate_out="g2", norm="norm", o="o")
        n.update(names or {})
        self.names = n
        self.channels = 2 * self.num_kv_heads * self.dim + self.num_heads * self.vdim   # what passes the convolution
        self.qkv = self.decay_in = self.gate_in = self.beta = self.in_proj = None
        self.conv = self.decay_log = self.decay_out = self.decay_bias = self.gate_out = self.norm = self.o_proj = None
        self.conv_f = self.coef_f = self.decay_out_f = self.decay_bias_f = self.gate_out_f = self.norm_f = None
        self.decay_rank = self.gate_rank = 0

    def weight_specs(self):
        n, C, H, G = self.names, self.hidden_size, self.num_heads, self.num_kv_heads
        kd, vd = G * self.dim, H * self.vdim
        r = free_size(MADE_UP_RANK)
        return [
            WeightSpec("qkv", (WeightSource(n["q"], (kd, C)), WeightSource(n["k"], (kd, C)), WeightSource(n["v"], (vd, C)))),
            WeightSpec("conv", (WeightSource(n["q_conv"], (kd, self.taps)), WeightSource(n["k_conv"], (kd, self.taps)),
                                WeightSource(n["v_conv"], (vd, self.taps)))),
            WeightSpec("decay_in", (WeightSource(n["decay_in"], (r, C)),)),
            WeightSpec("gate_in", (WeightSource(n["gate_in"], (r, C)),)),
            WeightSpec("beta", (WeightSource(n["beta"], (H, C)),)),
            WeightSpec("decay_out", (WeightSource(n["decay_out"], (H * self.dim, r)),)),
            WeightSpec("decay_bias", (WeightSource(n["decay_bias"], (H * self.dim,)),)),
            WeightSpec("decay_log", (WeightSource(n["decay_log"], (H,)),)),
            WeightSpec("gate_out", (WeightSource(n["gate_out"], (vd, r)),)),
            WeightSpec("norm", (WeightSource(n["norm"], (self.vdim,)),), init="ones"),
            WeightSpec("o_proj", (WeightSource(n["o"], (C, vd)),)),
        ]

    def materialize(self, device, dtype):
        self.decay_rank, self.gate_rank = self.decay_in.shape[0], self.gate_in.shape[0]
        if self.decay_out.shape[1] != self.decay_rank or self.gate_out.shape[1] != self.gate_rank:
            raise ValueError(f"gated delta rule: the low-rank pairs' inner sizes differ: {tuple(self.decay_in.shape)} / "
                             f"{tuple(self.decay_out.shape)}, {tuple(self.gate_in.shape)} / {tuple(self.gate_out.shape)}")
        # everything that reads the layer's input, as one matrix: q, k, v | decay | gate | beta
        self.in_proj = torch.cat([self.qkv, self.decay_in, self.gate_in, self.beta], dim=0).contiguous()
        self.qkv = self.decay_in = self.gate_in = self.beta = None
        self.conv_f = self.conv.float().contiguous()
        self.coef_f = torch.exp(self.decay_log.float()).contiguous()
        self.decay_out_f = self.decay_out.float().contiguous()
        self.decay_bias_f = self.decay_bias.float().contiguous()
        self.gate_out_f = self.gate_out.float().contiguous()
        self.norm_f = self.norm.float().contiguous()

    def state_spec(self):
        return StateSpec((self.num_heads, self.vdim, self.dim), torch.float32)

    def further_states(self):
        # the convolution's last inputs, kept as they were read (activations)
        return {"conv": StateSpec((self.taps - 1, self.channels), None)} if self.taps > 1 else {}

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        H, G, C3 = self.num_heads, self.num_kv_heads, self.channels
        kd = G * self.dim
        p = ops.linear(x, self.in_proj, out_dtype=ctx.dtype)
        qkv = torch.empty((ctx.T, C3), dtype=ctx.dtype, device=p.device)
        ops.short_conv(p[:, :C3], self.conv_f, cache.states.get("mixer.conv"), ctx.q_start, ctx.positions,
                       ctx.state_slots, qkv, ctx.B, residual=False, silu=True)
        at = C3
        g = ops.lowrank_up(p[:, at:at + self.decay_rank], self.decay_out_f, self.decay_bias_f, decay_coef=self.coef_f)
        at += self.decay_rank
        gate = ops.lowrank_up(p[:, at:at + self.gate_rank], self.gate_out_f)
        at += self.gate_rank
        o = _scan_out(ctx, H * self.vdim)
        ops.linear_scan(qkv[:, :kd], qkv[:, kd:2 * kd], qkv[:, 2 * kd:], g, None, self.coef_f, 0.0, cache.state,
                        ctx.q_start, ctx.positions, ctx.state_slots, o, ctx.B, num_heads=H, num_kv_heads=G, dim=self.dim,
                        vdim=self.vdim, beta=p[:, at:at + H], unit=True, q_scale=self.dim ** -0.5)
        y = ops.head_norm_gate(o, self.norm_f, gate, "sigmoid", self.eps, ctx.dtype, num_heads=H, vdim=self.vdim)
        return ops.linear(y, self.o_proj, out_dtype=ctx.dtype)


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, dim: int, vdim: int, tau: float, eps: float,
                 names: Optional[dict] = None):
        if num_heads <= 0 or not 0 < dim <= ops.LINEAR_SCAN_MAX_DIM or vdim <= 0 or not tau > 0:
            raise ValueError(f"gated linear attention: {num_heads} heads of {dim}/{vdim} (keys of up to "
                             f"{ops.LINEAR_SCAN_MAX_DIM}), tau {tau}")
        self.hidden_size, self.num_heads, self.dim, self.vdim = int(hidden_size), int(num_heads), int(dim), int(vdim)
        self.tau, self.eps = float(tau), float(eps)
        n = dict(q="q", k="k", v="v", g="g", decay_in="a1", decay_out="a2", decay_bias="a2.b", norm="norm", o="o")
        n.update(names or {})
        self.names = n
        self.qkvg = self.decay_in = self.in_proj = None
        self.decay_out = self.decay_bias = self.norm = self.o_proj = None
        self.coef_f = self.decay_out_f = self.decay_bias_f = self.norm_f = None
        self.decay_rank = 0

    def weight_specs(self):
        n, C, H = self.names, self.hidden_size, self.num_heads
        kd, vd = H * self.dim, H * self.vdim
        r = free_size(MADE_UP_RANK)
        return [
            WeightSpec("qkvg", (WeightSource(n["q"], (kd, C)), WeightSource(n["k"], (kd, C)), WeightSource(n["v"], (vd, C)),
                                WeightSource(n["g"], (vd, C)))),
            WeightSpec("decay_in", (WeightSource(n["decay_in"], (r, C)),)),
            WeightSpec("decay_out", (WeightSource(n["decay_out"], (kd, r)),)),
            WeightSpec("decay_bias", (WeightSource(n["decay_bias"], (kd,)),)),
            WeightSpec("norm", (WeightSource(n["norm"], (self.vdim,)),), init="ones"),
            WeightSpec("o_proj", (WeightSource(n["o"], (C, vd)),)),
        ]

    def materialize(self, device, dtype):
        self.decay_rank = self.decay_in.shape[0]
        if self.decay_out.shape[1] != self.decay_rank:
            raise ValueError(f"gated linear attention: the decay's low-rank pair is {tuple(self.decay_in.shape)} / "
                             f"{tuple(self.decay_out.shape)}")
        self.in_proj = torch.cat([self.qkvg, self.decay_in], dim=0).contiguous()
        self.qkvg = self.decay_in = None
        self.coef_f = torch.full((self.num_heads,), 1.0 / self.tau, dtype=torch.float32, device=self.in_proj.device)
        self.decay_out_f = self.decay_out.float().contiguous()
        self.decay_bias_f = self.decay_bias.float().contiguous()
        self.norm_f = self.norm.float().contiguous()

    def state_spec(self):
        return StateSpec((self.num_heads, self.vdim, self.dim), torch.float32)

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        H = self.num_heads
        kd, vd = H * self.dim, H * self.vdim
        p = ops.linear(x, self.in_proj, out_dtype=ctx.dtype)
        at = 2 * kd + 2 * vd
        # sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau)
        g = ops.lowrank_up(p[:, at:at + self.decay_rank], self.decay_out_f, self.decay_bias_f, decay_coef=self.coef_f,
                           decay_sign=-1.0)
        o = _scan_out(ctx, vd)
        ops.linear_scan(p[:, :kd], p[:, kd:2 * kd], p[:, 2 * kd:2 * kd + vd], g, None, self.coef_f, 0.0, cache.state,
                        ctx.q_start, ctx.positions, ctx.state_slots, o, ctx.B, num_heads=H, num_kv_heads=H, dim=self.dim,
                        vdim=self.vdim, unit=False, q_scale=self.dim ** -0.5)
        y = ops.head_norm_gate(o, self.norm_f, p[:, 2 * kd + vd:at], "silu", self.eps, ctx.dtype, num_heads=H,
                               vdim=self.vdim)
        return ops.linear(y, self.o_proj, out_dtype=ctx.dtype)


@MIXERS.register("time_mix")
class TimeMix(Mixer):
    """A matrix per head with a decay per key channel and a bonus for the current token, on inputs
    that are blends of a token's row with the row before it:

        for s in r, k, v, g, w:  x_s = x_t + (x_(t-1) - x_t) * mu_s       (x_(-1) = 0; the last row is part of the state)
        r = W_r x_r, k = W_k x_k (H heads of dim), v = W_v x_v (H heads of vdim), gate = silu(W_g x_g)
        decay = exp(-exp(W_w2 tanh(W_w1 x_w) + w0))                      one per head and key channel
        o = (S + diag(u) k v^T)^T r;  S <- diag(decay) S + k v^T          u: the bonus, per head and key channel
        y = W_o (concat_h(o_h / rms(o_h)) * w_norm * gate)               w_norm over all heads' values

    Blends and products run in the step's type; the decay (tanh, both exponentials), the recurrence,
    its state and the heads' norm are 32-bit.  The state is kept transposed, [heads, vdim, dim]."""

    def __init__(self, hidden_size: int, num_heads: int, dim: int, eps: float, vdim: Optional[int] = None,
                 names: Optional[dict] = None):
        vdim = dim if vdim is None else vdim
        if num_heads <= 0 or not 0 < dim <= ops.LINEAR_SCAN_MAX_DIM or vdim <= 0:
            raise ValueError(f"time mix: {num_heads} heads of {dim}/{vdim} (keys of up to {ops.LINEAR_SCAN_MAX_DIM})")
        self.hidden_size, self.num_heads, self.dim, self.vdim, self.eps = int(hidden_size), int(num_heads), int(dim), int(vdim), float(eps)
        n = dict(mu="mu.", r="r", k="k", v="v", g="g", decay_in="w1", decay_out="w2", decay_bias="w0", bonus="u",
                 norm="norm", o="o")
        n.update(names or {})
        self.names = n
        self.mu = self.r_proj = self.k_proj = self.v_proj = self.g_proj = self.decay_in = None
        self.decay_out = self.decay_bias = self.bonus = self.norm = self.o_proj = None
        self.mu_f = self.decay_out_f = self.decay_bias_f = self.bonus_f = self.norm_f = self.coef_f = None

    def weight_specs(self):
        n, C, H = self.names, self.hidden_size, self.num_heads
        kd, vd = H * self.dim, H * self.vdim
        rank = free_size(MADE_UP_RANK)
        return [
            WeightSpec("mu", tuple(WeightSource(n["mu"] + s, (C,)) for s in "rkvgw")),
            WeightSpec("r_proj", (WeightSource(n["r"], (kd, C)),)),
            WeightSpec("k_proj", (WeightSource(n["k"], (kd, C)),)),
            WeightSpec("v_proj", (WeightSource(n["v"], (vd, C)),)),
            WeightSpec("g_proj", (WeightSource(n["g"], (vd, C)),)),
            WeightSpec("decay_in", (WeightSource(n["decay_in"], (rank, C)),)),
            WeightSpec("decay_out", (WeightSource(n["decay_out"], (kd, rank)),)),
            WeightSpec("decay_bias", (WeightSource(n["decay_bias"], (kd,)),)),
            WeightSpec("bonus", (WeightSource(n["bonus"], (H, self.dim)),)),
            WeightSpec("norm", (WeightSource(n["norm"], (vd,)),), init="ones"),
            WeightSpec("o_proj", (WeightSource(n["o"], (C, vd)),)),
        ]

    def materialize(self, device, dtype):
        if self.decay_out.shape[1] != self.decay_in.shape[0]:
            raise ValueError(f"time mix: the decay's low-rank pair is {tuple(self.decay_in.shape)} / {tuple(self.decay_out.shape)}")
        self.mu_f = self.mu.float().reshape(5, self.hidden_size).contiguous()
        self.decay_out_f = self.decay_out.float().contiguous()
        self.decay_bias_f = self.decay_bias.float().contiguous()
        self.bonus_f = self.bonus.float().reshape(-1).contiguous()
        self.norm_f = self.norm.float().contiguous()
        self.coef_f = torch.ones(self.num_heads, dtype=torch.float32, device=self.mu.device)

    def state_spec(self):
        return StateSpec((self.num_heads, self.vdim, self.dim), torch.float32)

    def further_states(self):
        return {"shift": StateSpec((self.hidden_size,), None)}     # the previous token's input, as it was read

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        H = self.num_heads
        mixes = ops.shift_mix(x, self.mu_f, cache.states["mixer.shift"], ctx.q_start, ctx.positions, ctx.state_slots, ctx.B)
        r = ops.linear(mixes[0], self.r_proj, out_dtype=ctx.dtype)
        k = ops.linear(mixes[1], self.k_proj, out_dtype=ctx.dtype)
        v = ops.linear(mixes[2], self.v_proj, out_dtype=ctx.dtype)
        gate = ops.linear(mixes[3], self.g_proj, out_dtype=ctx.dtype)
        mid = ops.linear(mixes[4], self.decay_in, out_dtype=torch.float32)
        decay = ops.lowrank_up(mid, self.decay_out_f, self.decay_bias_f, mid_tanh=True, double_exp=True)
        o = _scan_out(ctx, H * self.vdim)
        ops.linear_scan(r, k, v, decay, None, self.coef_f, 0.0, cache.state, ctx.q_start, ctx.positions, ctx.state_slots,
                        o, ctx.B, num_heads=H, num_kv_heads=H, dim=self.dim, vdim=self.vdim, bonus=self.bonus_f)
        y = ops.head_norm_gate(o, self.norm_f, gate, "silu", self.eps, ctx.dtype, num_heads=H, vdim=self.vdim)
        return ops.linear(y, self.o_proj, out_dtype=ctx.dtype)


@MIXERS.register("selective_state_space")
class SelectiveStateSpace(Mixer):
    """A state-space layer with one decay per head and token, set by a step size:

        [z | x | B | C | dt] = W_in h           z, x: H heads of vdim; B, C: G groups of ``state`` values; dt: H
        x, B, C <- silu(causal convolution per channel (+ bias)), the last ``taps - 1`` inputs being part of the state
        dt <- softplus(dt + dt_bias);  per head (head h reads group h // (H / G)):
        S <- exp(-exp(A_log_h) dt) S + dt B x^T;   y = S^T C + D_h x
        out = W_o ( norm in ``norm_groups`` equal parts of (y * silu(z)) * w_norm )

    Products, the convolution and its silu run in the step's type (dt's product is kept in 32-bit);
    step sizes, decays, the recurrence, its state and the norm are 32-bit.  The state is kept
    transposed, [heads, vdim, state]."""

    def __init__(self, hidden_size: int, num_heads: int, vdim: int, state: int, groups: int, conv_taps: int,
                 norm_groups: int, eps: float, conv_bias: bool = True, names: Optional[dict] = None):
        if num_heads <= 0 or groups <= 0 or num_heads % groups:
            raise ValueError(f"{num_heads} heads do not split over {groups} groups")
        if not 0 < state <= ops.LINEAR_SCAN_MAX_DIM or vdim <= 0 or conv_taps < 1 or norm_groups < 1 or \
                (num_heads * vdim) % norm_groups:
            raise ValueError(f"state space: heads of {vdim}, {state} state values (up to {ops.LINEAR_SCAN_MAX_DIM}), "
                             f"{conv_taps} taps, {norm_groups} norm groups")
        self.hidden_size, self.num_heads, self.vdim, self.state, self.groups = int(hidden_size), int(num_heads), int(vdim), int(state), int(groups)
        self.taps, self.norm_groups, self.eps, self.has_conv_bias = int(conv_taps), int(norm_groups), float(eps), bool(conv_bias)
        self.inner = self.num_heads * self.vdim
        self.channels = self.inner + 2 * self.groups * self.state      # what passes the convolution
        n = dict(in_proj="in", conv="conv", conv_bias="conv.b", dt_bias="dt_bias", decay_log="A_log", skip="D", norm="norm", o="o")
        n.update(names or {})
        self.names = n
        self.in_proj = self.conv = self.conv_bias = self.dt_bias = self.decay_log = self.skip = self.norm = self.o_proj = None
        self.in_main = self.in_dt = None
        self.conv_f = self.conv_bias_f = self.dt_bias_f = self.coef_f = self.skip_f = self.norm_f = None

    def weight_specs(self):
        n, C, H = self.names, self.hidden_size, self.num_heads
        specs = [
            WeightSpec("in_proj", (WeightSource(n["in_proj"], (self.inner + self.channels + H, C)),)),
            WeightSpec("conv", (WeightSource(n["conv"], (self.channels, self.taps)),)),
            WeightSpec("dt_bias", (WeightSource(n["dt_bias"], (H,)),)),
            WeightSpec("decay_log", (WeightSource(n["decay_log"], (H,)),)),
            WeightSpec("skip", (WeightSource(n["skip"], (H,)),), init="ones"),
            WeightSpec("norm", (WeightSource(n["norm"], (self.inner,)),), init="ones"),
            WeightSpec("o_proj", (WeightSource(n["o"], (C, self.inner)),)),
        ]
        if self.has_conv_bias:
            specs.append(WeightSpec("conv_bias", (WeightSource(n["conv_bias"], (self.channels,)),)))
        return specs

    def materialize(self, device, dtype):
        main = self.inner + self.channels
        self.in_main = self.in_proj[:main].contiguous()
        self.in_dt = self.in_proj[main:].contiguous()
        self.in_proj = None
        self.conv_f = self.conv.float().contiguous()
        self.conv_bias_f = self.conv_bias.float().contiguous() if self.has_conv_bias else None
        self.dt_bias_f = self.dt_bias.float().contiguous()
        self.coef_f = torch.exp(self.decay_log.float()).contiguous()
        self.skip_f = self.skip.float().contiguous()
        self.norm_f = self.norm.float().contiguous()

    def state_spec(self):
        return StateSpec((self.num_heads, self.vdim, self.state), torch.float32)

    def further_states(self):
        return {"conv": StateSpec((self.taps - 1, self.channels), None)} if self.taps > 1 else {}

    def forward(self, ctx: StepContext, x, cache: LayerCache):
        H, G, inner, gn = self.num_heads, self.groups, self.inner, self.groups * self.state
        p = ops.linear(x, self.in_main, out_dtype=ctx.dtype)                 # z | x | B | C
        dt = ops.linear(x, self.in_dt, out_dtype=torch.float32)
        xbc = torch.empty((ctx.T, self.channels), dtype=ctx.dtype, device=p.device)
        ops.short_conv(p[:, inner:], self.conv_f, cache.states.get("mixer.conv"), ctx.q_start, ctx.positions,
                       ctx.state_slots, xbc, ctx.B, residual=False, silu=True, bias=self.conv_bias_f)
        o = _scan_out(ctx, inner)
        ops.linear_scan(xbc[:, inner + gn:], xbc[:, inner:inner + gn], xbc[:, :inner], dt, self.dt_bias_f, self.coef_f, 1.0,
                        cache.state, ctx.q_start, ctx.positions, ctx.state_slots, o, ctx.B, num_heads=H, num_kv_heads=G,
                        dim=self.state, vdim=self.vdim, z_per_head=True, key_step=True)
        y = ops.skip_gate_group_norm(o, xbc[:, :inner], self.skip_f, p[:, :inner], self.norm_f, self.norm_groups, self.eps,
                                     vdim=self.vdim)
        return ops.linear(y, self.o_proj, out_dtype=ctx.dtype)
