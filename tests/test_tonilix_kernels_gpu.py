"""The kernels behind Tonilix's mechanisms, each alone against the plain
implementation (tests/plain/tonilix_plain.py): the norm in groups with the
scaled branch it adds, the position vector, the token shift and the short
convolutions with their states over several steps and slots, both recurrences
with matrices carried from step to step, the heads' norm with its gates, the
low-rank projections, the biased projection with the query multiplier and its
page write, the gates and sums, and the router that chooses within groups with
the experts' products."""
import math

import numpy as np
import pytest
import torch

from plain import tonilix_plain as TP

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
DEV = "cuda:0"
F = torch.float64


def tdt(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


def close(got, want, dtype, what="", floor=1.0, tol=None):
    got, want = got.double().cpu(), want.double().cpu()
    tol = tol if tol is not None else (2e-5 if dtype == "float32" else 2e-2)
    scale = max(floor, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= tol * scale, f"{what}: max error {err:.3e} at scale {scale:.3f}"


def ints(a):
    return torch.tensor(np.asarray(a, dtype=np.int32), device=DEV)


@pytest.fixture(scope="module")
def ops():
    from lyapunov_engine_amd.kernels import ops as o
    return o


# ------------------------------------------------------------ norm in groups
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,groups", [(72, 3), (64, 1), (128, 4), (100, 5), (2048, 8), (40, 40), (2048, 2), (512, 1), (1024, 1), (9000, 3)])
def test_group_norm_adds_the_scaled_branch_first(ops, dtype, H, groups):
    T = 11
    g = torch.Generator().manual_seed(H + groups)
    h = torch.randn(T, H, generator=g) * 3
    d = (torch.randn(T, H, generator=g) * 2).to(tdt(dtype))
    s = torch.randn(H, generator=g)
    w = 1 + 0.3 * torch.randn(H, generator=g)
    hd = h.to(DEV)
    out = torch.empty(T, H, dtype=tdt(dtype), device=DEV)
    ops.group_rmsnorm(hd, w.to(DEV), groups, 1e-5, out, delta=d.to(DEV), scale=s.to(DEV))
    summed = h.double() + d.double() * s.double()
    close(hd, summed, "float32", "the stream after the sum")
    close(out, TP.group_rms_norm(summed, w.double(), 1e-5, groups), dtype, "normed rows")
    # float partial sums, and picked rows that leave the stream alone
    parts = torch.randn(3, T, H, generator=g)
    hd2 = h.to(DEV)
    out32 = torch.empty(T, H, dtype=torch.float32, device=DEV)
    ops.group_rmsnorm(hd2, w.to(DEV), groups, 1e-5, out32, delta=parts.to(DEV), scale=s.to(DEV))
    summed2 = h.double() + parts.double().sum(0) * s.double()
    close(out32, TP.group_rms_norm(summed2, w.double(), 1e-5, groups), "float32", "partial sums")
    rows = ints([7, 0, 3])
    picked = torch.empty(3, H, dtype=torch.float32, device=DEV)
    before = hd2.clone()
    ops.group_rmsnorm(hd2, w.to(DEV), groups, 1e-5, picked, rows=rows)
    assert torch.equal(hd2, before)
    close(picked, TP.group_rms_norm(summed2, w.double(), 1e-5, groups)[[7, 0, 3]], "float32", "picked rows")


def test_group_norm_of_unequal_groups_differs_from_one_norm(ops):
    """A row whose groups differ a thousandfold: one norm over the row would all but erase the small group."""
    h = torch.cat([torch.full((1, 8), 1000.0), torch.full((1, 8), 1.0)], 1)
    out = torch.empty(1, 16, dtype=torch.float32, device=DEV)
    ops.group_rmsnorm(h.to(DEV), torch.ones(16, device=DEV), 2, 0.0, out)
    assert torch.allclose(out.cpu(), torch.ones(1, 16), atol=1e-6)


def test_position_vector_far_out(ops):
    for H in (6, 72, 128):
        pos = [0, 1, 2, 63, 64, 1000, 4097, 100000]
        h = torch.zeros(len(pos), H, device=DEV)
        ops.add_sinusoid(h, ints(pos), 10000.0)
        want = TP.sinusoid(pos, H)
        assert float((h.double().cpu() - want).abs().max()) < 2e-6, H


# ----------------------------------------------- filters over time with state
def conv_steps(ops, dtype, x, w, cuts, silu, C_lo=0, C_hi=None):
    """One request's rows fed in the given portions through ``ops.short_conv`` with a state slot."""
    T, C = x.shape
    taps = w.shape[1]
    state = torch.full((3, max(taps - 1, 1), C), 7.0, dtype=tdt(dtype), device=DEV)   # a slot someone left
    outs, at = [], 0
    for n in cuts:
        xs = x[at:at + n].to(tdt(dtype)).to(DEV)
        out = torch.empty_like(xs)
        ops.short_conv(xs, w.float().to(DEV), state if taps > 1 else None, ints([0, n]), ints(range(at, at + n)), ints([2]),
                       out, 1, residual=False, silu=silu)
        outs.append(out)
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 5])
def test_short_convolution_with_silu_over_steps(ops, dtype, taps):
    g = torch.Generator().manual_seed(taps)
    T, C = 29, 88
    x = torch.randn(T, C, generator=g).to(tdt(dtype)).double()
    w = torch.randn(C, taps, generator=g)
    want = TP.silu(TP.causal_conv(x, w.double()))
    for cuts in ([T], [1] * T, [2, 1, 7, 2, 1, 1, 15], [taps, 1, T - taps - 1]):
        close(conv_steps(ops, dtype, x, w, cuts, True), want, dtype, f"taps {taps}, portions {cuts[:4]}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift_is_its_two_tap_filter(ops, dtype):
    from lyapunov_engine_amd.parts.filters import TokenShift

    C, T = 72, 17
    g = torch.Generator().manual_seed(5)
    part = TokenShift(C, tensor="")
    part.mix = torch.rand(C, generator=g).to(DEV)
    part.materialize(DEV, tdt(dtype))
    x = torch.randn(T, C, generator=g).to(tdt(dtype)).double()
    want = TP.token_shift(x, part.mix.double().cpu())
    for cuts in ([T], [1] * T, [2, 2, 1, 12]):
        close(conv_steps(ops, dtype, x, part.weight_f.cpu(), cuts, False), want, dtype, f"portions {cuts[:4]}")


def test_filters_of_two_requests_keep_to_their_slots(ops):
    """Two requests in one step, one continuing and one starting, with their slots swapped in order."""
    C, taps = 24, 3
    g = torch.Generator().manual_seed(1)
    w = torch.randn(C, taps, generator=g)
    a, b = torch.randn(9, C, generator=g), torch.randn(6, C, generator=g)
    state = torch.zeros(4, taps - 1, C, device=DEV)
    out = torch.empty(5, C, device=DEV)
    ops.short_conv(a[:5].to(DEV), w.to(DEV), state, ints([0, 5]), ints(range(5)), ints([3]), out, 1, residual=False)
    x = torch.cat([b, a[5:]]).to(DEV)
    out = torch.empty(10, C, device=DEV)
    ops.short_conv(x, w.to(DEV), state, ints([0, 6, 10]), ints(list(range(6)) + list(range(5, 9))), ints([1, 3]), out, 2,
                   residual=False)
    close(out[:6], TP.causal_conv(b.double(), w.double()), "float32", "the starting request")
    close(out[6:], TP.causal_conv(a.double(), w.double())[5:], "float32", "the continuing request")


# ---------------------------------------------------------------- recurrences
def scan_inputs(seed, T, H, G, D, V, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(T, G * D, generator=g).to(tdt(dtype))
    k = torch.randn(T, G * D, generator=g).to(tdt(dtype))
    v = torch.randn(T, H * V, generator=g).to(tdt(dtype))
    z = torch.randn(T, H * D, generator=g) * 2
    zb = torch.randn(H * D, generator=g)
    beta = (torch.randn(T, H, generator=g) * 2).to(tdt(dtype))
    return q, k, v, z, zb, beta


def run_scan(ops, cuts, q, k, v, z, zb, coef, sign, beta, H, G, D, V, unit, q_scale, slot=1, slots=3):
    state = torch.full((slots, H, V, D), 3.0, device=DEV)        # what another request left behind
    outs, at = [], 0
    for n in cuts:
        sl = slice(at, at + n)
        o = torch.empty(n, H * V, device=DEV)
        ops.linear_scan(q[sl].to(DEV), k[sl].to(DEV), v[sl].to(DEV), z[sl].to(DEV), zb.to(DEV) if zb is not None else None,
                        coef.to(DEV), sign, state, ints([0, n]), ints(range(at, at + n)), ints([slot]), o, 1, num_heads=H,
                        num_kv_heads=G, dim=D, vdim=V, beta=beta[sl].to(DEV) if beta is not None else None, unit=unit,
                        q_scale=q_scale)
        outs.append(o)
        at += n
    return torch.cat(outs), state


SCAN_SIZES = [(4, 2, 24, 10), (1, 1, 32, 48), (2, 2, 128, 16), (3, 1, 7, 5), (2, 1, 200, 8), (6, 3, 64, 64), (2, 2, 16, 130), (1, 1, 300, 6), (2, 1, 8, 3), (2, 2, 4, 70)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V", SCAN_SIZES)
def test_gated_delta_rule_over_steps(ops, dtype, H, G, D, V):
    T = 45
    q, k, v, z, zb, beta = scan_inputs(H * 7 + D, T, H, G, D, V, dtype)
    coef = torch.exp(torch.randn(H, generator=torch.Generator().manual_seed(2)) * 0.7)
    qd, kd = q.double().view(T, G, D), k.double().view(T, G, D)
    qd = qd / torch.sqrt((qd * qd).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kd = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + 1e-6)
    qd, kd = qd.repeat_interleave(H // G, 1), kd.repeat_interleave(H // G, 1)
    gd = torch.exp(-coef.double()[None, :, None] * TP.softplus(z.double() + zb.double()).view(T, H, D))
    want, S = TP.delta_rule_scan(qd, kd, v.double().view(T, H, V), gd, torch.sigmoid(beta.double()))
    for cuts in ([T], [1] * T, [2, 1, 9, 8, 17, 2, 6], [8, 8, 8, 21]):
        got, state = run_scan(ops, cuts, q, k, v, z, zb, coef, 1.0, beta, H, G, D, V, True, D ** -0.5)
        close(got, want.reshape(T, H * V), dtype, f"outputs, portions {cuts[:4]}", floor=0.1, tol=5e-5 if dtype == "float32" else 2e-2)
        close(state[1], S.transpose(1, 2), "float32", f"the slot's matrices, portions {cuts[:4]}", floor=0.1, tol=5e-5)
        assert float((state[0] - 3.0).abs().max()) == 0.0 and float((state[2] - 3.0).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,V", SCAN_SIZES)
@pytest.mark.parametrize("tau", [1.0, 16.0])
def test_gated_linear_attention_over_steps(ops, dtype, H, G, D, V, tau):
    G = H
    T = 45
    q, k, v, z, zb, _ = scan_inputs(H * 5 + V, T, H, G, D, V, dtype)
    coef = torch.full((H,), 1.0 / tau)
    a = torch.pow(torch.sigmoid(z.double() + zb.double()), 1.0 / tau).view(T, H, D)
    want, S = TP.decayed_outer_scan(q.double().view(T, H, D) * D ** -0.5, k.double().view(T, H, D), v.double().view(T, H, V), a)
    for cuts in ([T], [1] * T, [3, 2, 25, 15]):
        got, state = run_scan(ops, cuts, q, k, v, z, zb, coef, -1.0, None, H, G, D, V, False, D ** -0.5)
        close(got, want.reshape(T, H * V), dtype, f"outputs, portions {cuts[:4]}", tol=5e-5 if dtype == "float32" else 2e-2)
        close(state[1], S.transpose(1, 2), "float32", f"the slot's matrices, portions {cuts[:4]}", tol=5e-5)


@pytest.mark.parametrize("H,G,D,V", [(4, 2, 24, 10), (2, 2, 128, 16), (1, 1, 300, 6)])
def test_recurrences_take_decays_worked_out_by_the_low_rank_kernel(ops, H, G, D, V):
    """The path the mixers take: the second half of the decay's low-rank pair hands on exp(-coef softplus(sign y))
    itself, and the recurrence is told so (sign 0).  Long enough for several chunks."""
    T, R = 150, 6
    q, k, v, _, zb, beta = scan_inputs(H + D, T, H, G, D, V, "float32")
    g = torch.Generator().manual_seed(9)
    mid, w = torch.randn(T, R, generator=g), torch.randn(H * D, R, generator=g)
    coef = torch.exp(torch.randn(H, generator=g) * 0.7)
    y = mid.double() @ w.double().T + zb.double()
    for sign, with_beta in ((1.0, True), (-1.0, False)):
        dec = ops.lowrank_up(mid.to(DEV), w.to(DEV), zb.to(DEV), decay_coef=coef.to(DEV), decay_sign=sign)
        gd = torch.exp(-coef.double()[None, :, None] * TP.softplus(sign * y).view(T, H, D))
        close(dec, gd.reshape(T, H * D), "float32", "decays", tol=2e-6)
        qd = q.double().view(T, G, D).repeat_interleave(H // G, 1)
        kd = k.double().view(T, G, D).repeat_interleave(H // G, 1)
        if with_beta:
            want, _ = TP.delta_rule_scan(qd * 0.3, kd * 0.1, v.double().view(T, H, V), gd, torch.sigmoid(beta.double()))
        else:
            want, _ = TP.decayed_outer_scan(qd * 0.3, kd * 0.1, v.double().view(T, H, V), gd)
        for cuts in ([T], [70, 1, 33, 46]):
            got, _ = run_scan(ops, cuts, q, k * 0.1, v, dec.cpu(), None, coef, 0.0, beta if with_beta else None, H, G, D, V,
                              False, 0.3)
            close(got, want.reshape(T, H * V), "float32", f"sign {sign}, portions {cuts}", floor=0.1, tol=5e-5)


def test_recurrence_keeps_one_early_write_for_hundreds_of_tokens(ops):
    """Decays of nearly one, keys that are all alike but the first, which is at right angles to them: the
    first value is still read, exactly, by a query along the first key 600 tokens later."""
    H, D, V, T = 1, 16, 8, 600
    k = torch.zeros(T, D)
    k[0, 3] = 1.0
    k[1:, 5] = 1.0
    v = torch.randn(T, V, generator=torch.Generator().manual_seed(0))
    q = torch.zeros(T, D)
    q[:, 3] = 1.0
    z = torch.full((T, D), 30.0)            # sigmoid(30)^(1/tau) is 1 to nine places
    coef = torch.ones(H)
    for cuts in ([T], [300, 1, 1, 298], [7] * 85 + [5]):
        got, _ = run_scan(ops, cuts, q, k, v, z, None, coef, -1.0, None, H, H, D, V, False, 1.0)
        close(got[-1], v[0].double(), "float32", "the first value at the end", tol=1e-5)
    # the delta rule with beta = 1 replaces what a key holds: the second write to key 5 removes the first
    beta = torch.full((T, H), 40.0)
    zz = torch.full((T, D), -40.0)          # exp(-softplus(-40)) is 1
    q2 = torch.zeros(T, D)
    q2[:, 5] = 1.0
    got, _ = run_scan(ops, [T], q2, k, v, zz, None, coef, 1.0, beta, H, H, D, V, False, 1.0)
    close(got[-1], v[-1].double(), "float32", "the last write to a key is what it holds", tol=1e-5)
    close(got[0], torch.zeros(V).double(), "float32", "a key at right angles reads nothing", tol=1e-5)


def test_recurrences_of_several_requests_in_one_step(ops):
    """Three requests of unequal length in one step, one of them continuing from its slot, against each alone."""
    H, G, D, V = 4, 2, 24, 12
    dtype = "float32"
    lens = [9, 1, 14]
    data = [scan_inputs(10 + i, n, H, G, D, V, dtype) for i, n in enumerate(lens)]
    coef = torch.tensor([0.5, 1.0, 2.0, 0.1])
    alone = [run_scan(ops, [n], *d[:5], coef, 1.0, d[5], H, G, D, V, True, 0.2)[0] for n, d in zip(lens, data)]
    state = torch.full((5, H, V, D), 9.0, device=DEV)
    first = 4                                   # request 0 has run its first 4 rows in an earlier step, in slot 4
    d0 = data[0]
    o = torch.empty(first, H * V, device=DEV)
    ops.linear_scan(d0[0][:first].to(DEV), d0[1][:first].to(DEV), d0[2][:first].to(DEV), d0[3][:first].to(DEV), d0[4].to(DEV),
                    coef.to(DEV), 1.0, state, ints([0, first]), ints(range(first)), ints([4]), o, 1, num_heads=H, num_kv_heads=G,
                    dim=D, vdim=V, beta=d0[5][:first].to(DEV), unit=True, q_scale=0.2)
    cat = lambda i: torch.cat([data[0][i][first:], data[1][i], data[2][i]]).to(DEV)
    n0 = lens[0] - first
    out = torch.empty(n0 + lens[1] + lens[2], H * V, device=DEV)
    pos = list(range(first, lens[0])) + [0] + list(range(lens[2]))
    # every request has its own decay bias in this test's data; the kernel takes one: fold it into z
    zfold = torch.cat([data[0][3][first:] + data[0][4], data[1][3] + data[1][4], data[2][3] + data[2][4]]).to(DEV)
    ops.linear_scan(cat(0), cat(1), cat(2), zfold, None, coef.to(DEV), 1.0, state, ints([0, n0, n0 + 1, n0 + 1 + lens[2]]),
                    ints(pos), ints([4, 0, 2]), out, 3, num_heads=H, num_kv_heads=G, dim=D, vdim=V, beta=cat(5), unit=True,
                    q_scale=0.2)
    close(out[:n0], alone[0][first:], dtype, "the continuing request", tol=5e-5)
    close(out[n0:n0 + 1], alone[1], dtype, "the request of one token", tol=5e-5)
    close(out[n0 + 1:], alone[2], dtype, "the starting request", tol=5e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["sigmoid", "silu"])
@pytest.mark.parametrize("H,V", [(4, 10), (1, 48), (3, 128), (2, 200)])
def test_heads_norm_and_gate(ops, dtype, kind, H, V):
    T = 13
    g = torch.Generator().manual_seed(H + V)
    o = torch.randn(T, H * V, generator=g) * 5
    w = 1 + 0.3 * torch.randn(V, generator=g)
    wide = torch.randn(T, H * V + 9, generator=g) * 2
    for gate_dtype in {"float32", dtype}:
        gate = wide.to(tdt(gate_dtype))
        got = ops.head_norm_gate(o.to(DEV), w.to(DEV), gate.to(DEV)[:, 5:5 + H * V], kind, 1e-5, tdt(dtype), num_heads=H, vdim=V)
        gd = gate.double()[:, 5:5 + H * V].view(T, H, V)
        act = torch.sigmoid(gd) if kind == "sigmoid" else TP.silu(gd)
        close(got, TP.head_rms_gate(o.double().view(T, H, V), w.double(), 1e-5, act).reshape(T, H * V), dtype, kind)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,N,R", [(1, 96, 5), (9, 40, 7), (70, 512, 16), (8, 33, 1)])
def test_low_rank_second_half_in_32_bit(ops, dtype, T, N, R):
    g = torch.Generator().manual_seed(N)
    wide = torch.randn(T, R + 11, generator=g).to(tdt(dtype))
    w, b = torch.randn(N, R, generator=g), torch.randn(N, generator=g)
    got = ops.lowrank_up(wide.to(DEV)[:, 4:4 + R], w.to(DEV), b.to(DEV))
    assert got.dtype == torch.float32
    close(got, wide.double()[:, 4:4 + R] @ w.double().T + b.double(), "float32", "with bias")
    close(ops.lowrank_up(wide.to(DEV)[:, 4:4 + R], w.to(DEV)), wide.double()[:, 4:4 + R] @ w.double().T, "float32", "without")


# ----------------------------------------- projections, gates and sums of the pair
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 1, 24, 20), (2, 2, 32, 32), (3, 1, 7, 5), (8, 2, 64, 64)])
@pytest.mark.parametrize("coef,every", [(0.7, 5), (1.0, 1), (0.25, 64)])
def test_biased_projection_multiplier_and_page_write(ops, dtype, sizes, coef, every):
    H, G, D, V = sizes
    page = 4
    g = torch.Generator().manual_seed(H * 100 + D + every)
    # positions on both sides of the places where floor((p + 1) / every) steps, near and far out
    pos = [0, every - 2 if every > 2 else 0, every - 1, every, 2 * every - 2, 2 * every - 1, 40, 777 * every - 1, 777 * every - 2, 5]
    pos = [max(p, 0) for p in pos]
    T = len(pos)
    n = (H + G) * D + G * V
    pre = torch.randn(T, n + 6, generator=g) * 2
    bias = torch.randn(n, generator=g)
    slots = torch.tensor([8, 9, 10, 11, 0, 1, 2, 5, 6, -1], dtype=torch.int32)      # the last row is padding
    kpool = torch.zeros(3, G, page, D, dtype=tdt(dtype), device=DEV)
    vpool = torch.zeros(3, G, V, page, dtype=tdt(dtype), device=DEV)
    q = ops.qkv_bias_temper_kv(pre.to(DEV)[:, :n + 6], bias.to(DEV), ints(pos), coef, every, slots.to(DEV), kpool, vpool,
                               tdt(dtype), num_heads=H, num_kv_heads=G, dim=D, vdim=V, page_size=page)
    x = pre.double()[:, :n] + bias.double()
    mult = torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in pos], dtype=F)
    close(q, x[:, :H * D] * mult[:, None], dtype, "queries")
    k, v = x[:, H * D:(H + G) * D].view(T, G, D), x[:, (H + G) * D:].view(T, G, V)
    for t in range(T - 1):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        close(kpool[p, :, o, :], k[t], dtype, f"key of row {t}")
        close(vpool[p, :, :, o], v[t], dtype, f"value of row {t}")
    assert float(kpool[1, :, 3, :].abs().max()) == 0.0 and float(kpool[0, :, 3, :].abs().max()) == 0.0, \
        "slots nobody named stay as they were"


@pytest.mark.parametrize("dtype", DTYPES)
def test_gates_and_sums(ops, dtype):
    g = torch.Generator().manual_seed(3)
    T, N = 7, 90
    x = torch.randn(T, N, generator=g).to(tdt(dtype))
    wide = torch.randn(T, N + 10, generator=g) * 3
    for kind, act in (("sigmoid", torch.sigmoid), ("silu", TP.silu)):
        for gd in {"float32", dtype}:
            gate = wide.to(tdt(gd))
            got = ops.gate_mul(x.clone().to(DEV), gate.to(DEV)[:, 3:3 + N], kind)
            close(got, x.double() * act(gate.double()[:, 3:3 + N]), dtype, f"{kind} gate")
    gu = (torch.randn(T, 2 * N, generator=g) * 3).to(tdt(dtype))
    close(ops.glu_act(gu.to(DEV), "gelu_tanh"), TP.gelu_tanh(gu.double()[:, :N]) * gu.double()[:, N:], dtype, "gelu gate")
    close(ops.glu_act(gu.to(DEV), "silu"), TP.silu(gu.double()[:, :N]) * gu.double()[:, N:], dtype, "silu gate")
    a, b = torch.randn(T, N, generator=g), torch.randn(T, N, generator=g).to(tdt(dtype))
    bias = torch.randn(N, generator=g)
    got = ops.weighted_sum(a.to(DEV), 0.8, b.to(DEV), -1.5, bias.to(DEV))
    assert got.dtype == torch.float32 and tuple(got.shape) == (1, T, N)
    close(got[0], 0.8 * (a.double() + bias.double()) - 1.5 * b.double(), "float32", "weighted sum")


# -------------------------------------------------------------------- experts
ROUTERS = [dict(experts=6, top=2, scale=1.5, groups=dict(count=3, keep=2)), dict(experts=4, top=1, scale=1.0, groups=dict(count=4, keep=4)),
           dict(experts=8, top=3, scale=2.0, groups=dict(count=2, keep=1)), dict(experts=72, top=5, scale=3.0, groups=dict(count=9, keep=4)),
           dict(experts=1, top=1, scale=0.9, groups=dict(count=1, keep=1)), dict(experts=64, top=8, scale=2.5, groups=dict(count=8, keep=4)),
           dict(experts=12, top=4, scale=1.0, groups=dict(count=1, keep=1)), dict(experts=256, top=8, scale=2.5, groups=dict(count=8, keep=4))]


@pytest.mark.parametrize("cores", [True, False], ids=["matrix cores", "plain sums"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("r", ROUTERS, ids=lambda r: f"{r['top']}of{r['experts']}in{r['groups']['keep']}of{r['groups']['count']}")
def test_router_chooses_within_the_best_groups(ops, dtype, r, cores):
    E, top = r["experts"], r["top"]
    T, K = 50, 40
    g = torch.Generator().manual_seed(E)
    x = torch.randn(T, K, generator=g).to(tdt(dtype))
    W = torch.randn(E, K, generator=g) * 0.5
    corr = torch.randn(E, generator=g) * 0.6 - 0.8          # many choice scores are negative
    idx, wgt = ops.moe_route_grouped(x.to(DEV), W.to(DEV), corr.to(DEV), top, r["groups"]["count"], r["groups"]["keep"], r["scale"],
                                     on_matrix_cores=cores)
    s = torch.sigmoid(x.double() @ W.double().T)
    margins = []
    chosen, weights = TP.choose_experts(s, corr.double(), r, margins)
    clear = margins[0] > 1e-4
    assert int(clear.sum()) > T // 2
    got = torch.sort(idx.cpu().long(), -1).values
    assert torch.equal(got[clear], torch.sort(chosen, -1).values[clear])
    # weights: the plain scores of whatever was chosen, over their sum, times the scale
    want = TP.route_weights(s, idx.cpu().long(), r)
    close(wgt, want, "float32", "weights", tol=1e-5)
    assert torch.allclose(wgt.sum(-1).cpu().double(), torch.full((T,), r["scale"], dtype=F), atol=1e-4)


def test_router_shuts_groups_out_even_when_all_choice_scores_are_negative(ops):
    """Scores set by hand through a router that reads one-hot rows.  Two groups of three, one kept, two
    chosen.  All choice scores are negative; the kept group's second expert is below every expert of the
    other group, and is still chosen: shut-out experts count as minus infinity, not as nought."""
    r = dict(experts=6, top=2, scale=1.0, groups=dict(count=2, keep=1))
    logits = torch.tensor([[2.0, -3.0, -4.0, 1.0, 0.5, -5.0]])
    corr = torch.full((6,), -1.5)
    x = torch.tensor([[1.0]])
    idx, wgt = ops.moe_route_grouped(x.to(DEV), logits.T.contiguous().to(DEV), corr.to(DEV), 2, 2, 1, 1.0)
    s = torch.sigmoid(logits.double())
    chosen, weights = TP.choose_experts(s, corr.double(), r)
    # group scores: (0.88 - 1.5) + (0.047 - 1.5) = -2.07 against (0.73 - 1.5) + (0.62 - 1.5) = -1.65: the second group
    assert sorted(chosen[0].tolist()) == [3, 4] and sorted(idx[0].tolist()) == [3, 4]
    logits2 = torch.tensor([[4.0, -3.0, -4.0, 1.0, 0.5, -5.0]])
    corr2 = torch.tensor([-1.2, -1.5, -1.5, -1.5, -1.5, -1.5])       # group scores -1.67 against -1.65 ... still the second
    idx2, _ = ops.moe_route_grouped(x.to(DEV), logits2.T.contiguous().to(DEV), corr2.to(DEV), 2, 2, 1, 1.0)
    chosen2, _ = TP.choose_experts(torch.sigmoid(logits2.double()), corr2.double(), r)
    assert sorted(idx2[0].tolist()) == sorted(chosen2[0].tolist())
    corr3 = torch.tensor([0.0, -1.5, -1.5, -1.5, -1.5, -1.5])        # now the first group, whose second best is far below
    idx3, wgt3 = ops.moe_route_grouped(x.to(DEV), logits2.T.contiguous().to(DEV), corr3.to(DEV), 2, 2, 1, 1.0)
    chosen3, w3 = TP.choose_experts(torch.sigmoid(logits2.double()), corr3.double(), r)
    assert sorted(chosen3[0].tolist()) == [0, 1] and sorted(idx3[0].tolist()) == [0, 1]
    order = torch.argsort(idx3[0].cpu())
    close(wgt3[0].cpu()[order], w3[0][torch.argsort(chosen3[0])], "float32", "weights without the correction", tol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,I,K,T", [(6, 2, 40, 72, 33), (1, 1, 56, 40, 5), (8, 3, 64, 128, 200), (72, 5, 8, 64, 17), (4, 2, 100, 100, 1)])
def test_experts_products_and_weighted_sum(ops, dtype, E, top, I, K, T):
    g = torch.Generator().manual_seed(E * 10 + top)
    x = (torch.randn(T, K, generator=g)).to(tdt(dtype))
    up = (torch.randn(E, I, K, generator=g) * K ** -0.5).to(tdt(dtype))
    down = (torch.randn(E, K, I, generator=g) * I ** -0.5).to(tdt(dtype))
    idx = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wgt = torch.rand(T, top, generator=g)
    plan = ops.moe_sort(idx.to(DEV), E)
    act = ops.moe_gemm(x.to(DEV), up.to(DEV), plan, gated=False, gather=True, relu2=True)
    y = ops.moe_gemm(act, down.to(DEV), plan, gated=False)
    out = ops.moe_combine(y, plan, wgt.to(DEV), T)
    want = torch.zeros(T, K, dtype=F)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            want[t] += wgt[t, j].double() * ((torch.relu(x[t].double() @ up[e].double().T) ** 2) @ down[e].double().T)
    got = out.sum(0) if out.dim() == 3 else out
    close(got, want, dtype, "experts", tol=2e-5 if dtype == "float32" else 3e-2)
