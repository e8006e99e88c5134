"""The kernels behind Vobotar's mechanisms, each alone against the plain
implementation (tests/plain/vobotar_plain.py): what stands between an attention
layer's projection and its pages (biases, the norms per head and over a whole
projection, both rotations, values that are the keys, blended values);
attention with capped scores, a distance penalty, sinks and windows on all three
kernels over shuffled pages, with single keys made to carry the result just
inside and just outside a window; the blends with the previous row and their
state; both new forms of the recurrence; and the small row-wise kernels."""
import math

import numpy as np
import pytest
import torch

from plain import vobotar_plain as VP

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


# ------------------------------------------- from the projection to the pages
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(3, 1, 10, 12, 6), (4, 2, 32, 32, 32), (2, 2, 7, 5, 4), (5, 5, 16, 24, 0), (8, 2, 64, 64, 16)])
@pytest.mark.parametrize("norm", ["none", "head", "head bare", "whole"])
@pytest.mark.parametrize("pairing", ["neighbours", "halves"])
def test_bias_norm_rotation_and_page_write(dtype, sizes, norm, pairing):
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.rope import RotaryEncoding

    H, G, D, V, rot = sizes
    T, page = 9, 4
    g = torch.Generator().manual_seed(H * 100 + D)
    n = (H + G) * D + G * V
    pre = torch.randn(T, n + 3, generator=g) * 2                      # three more columns that are not ours
    bias = torch.randn(n, generator=g)
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 42, 777, 5], dtype=torch.int32)
    slots = torch.tensor([8, 9, 10, 11, 0, 1, 2, 5, -1], dtype=torch.int32)      # the last row is padding
    mode = norm.split()[0]
    wq = wk = None
    if norm == "head":
        wq, wk = 1 + 0.3 * torch.randn(D, generator=g), 1 + 0.3 * torch.randn(D, generator=g)
    elif norm == "whole":
        wq, wk = 1 + 0.3 * torch.randn(H * D, generator=g), 1 + 0.3 * torch.randn(G * D, generator=g)
    table = None
    if rot:
        enc = RotaryEncoding(rot, 300.0, 1024, precise=True)
        enc.materialize(DEV, tdt(dtype))
        table = enc.table
    kpool = torch.zeros(3, G, page, D, dtype=tdt(dtype), device=DEV)
    vpool = torch.zeros(3, G, V, page, dtype=tdt(dtype), device=DEV)
    d = lambda t: None if t is None else t.to(DEV)
    q, kept = ops.qkv_prepare(pre.to(DEV), tdt(dtype), num_heads=H, num_kv_heads=G, dim=D, vdim=V, slots=slots.to(DEV),
                              kpool=kpool, vpool=vpool, page_size=page, bias=bias.to(DEV), norm=mode, q_weight=d(wq), k_weight=d(wk),
                              eps=1e-5, positions=pos.to(DEV), table=table, pairing=pairing, keep_values=True)
    x = (pre[:, :n] + bias).double()
    qq, kk, vv = x[:, :H * D], x[:, H * D:(H + G) * D], x[:, (H + G) * D:].reshape(T, G, V)
    if mode == "whole":
        qq, kk = VP.norm_plain(qq, wq.double(), 1e-5), VP.norm_plain(kk, wk.double(), 1e-5)
    qq, kk = qq.reshape(T, H, D), kk.reshape(T, G, D)
    if mode == "head":
        qq, kk = qq / VP.rms(qq, 1e-5), kk / VP.rms(kk, 1e-5)
        if wq is not None:
            qq, kk = qq * wq.double(), kk * wk.double()
    if rot:
        turn = VP.rotate_neighbours if pairing == "neighbours" else VP.rotate_halves
        qq, kk = turn(qq, pos.tolist(), rot, 300.0), turn(kk, pos.tolist(), rot, 300.0)
    close(q.view(T, H, D), qq, dtype, "queries")
    close(kept.view(T, G, V), vv, "float32", "kept values")
    for t in range(T - 1):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        close(kpool[p, :, o], kk[t], dtype, f"keys of row {t}")
        close(vpool[p, :, :, o], vv[t], dtype, f"values of row {t}")
    assert float(kpool[1, :, 2:].abs().max()) == 0.0 and float(kpool[0, :, 3].abs().max()) == 0.0   # nothing for the padded row


@pytest.mark.parametrize("dtype", DTYPES)
def test_values_that_are_the_keys_and_blended_values(dtype):
    from lyapunov_engine_amd.kernels import ops

    H, G, D, T, page = 4, 2, 12, 6, 8
    g = torch.Generator().manual_seed(4)
    pre = torch.randn(T, (H + G) * D, generator=g)
    bias = torch.randn((H + G) * D, generator=g)
    slots = ints(np.arange(T))
    kpool = torch.zeros(1, G, page, D, dtype=tdt(dtype), device=DEV)
    vpool = torch.zeros(1, G, D, page, dtype=tdt(dtype), device=DEV)
    ops.qkv_prepare(pre.to(DEV), tdt(dtype), num_heads=H, num_kv_heads=G, dim=D, vdim=D, slots=slots, kpool=kpool, vpool=vpool,
                    page_size=page, bias=bias.to(DEV), norm="head", eps=1e-6, values_from_keys=True)
    k = (pre + bias).double()[:, H * D:].reshape(T, G, D)
    close(vpool[0, :, :, :T].permute(2, 0, 1), k, dtype, "the values are the biased keys before their norm")
    close(kpool[0, :, :T].permute(1, 0, 2), k / VP.rms(k, 1e-6), dtype, "the keys are normed")
    # blending: (1 - m) own + m other, with m on the device
    V = 10
    pre = torch.randn(T, (H + G) * D + G * V, generator=g)
    other = torch.randn(T, G * V, generator=g)
    vpool = torch.zeros(1, G, V, page, dtype=tdt(dtype), device=DEV)
    for m in (0.0, 0.3, 1.0):
        ops.qkv_prepare(pre.to(DEV), tdt(dtype), num_heads=H, num_kv_heads=G, dim=D, vdim=V, slots=slots, kpool=kpool, vpool=vpool,
                        page_size=page, blend=torch.tensor([m], device=DEV), other_values=other.to(DEV))
        want = (1 - m) * pre[:, (H + G) * D:].double() + m * other.double()
        close(vpool[0, :, :, :T].permute(2, 0, 1).reshape(T, G * V), want, dtype, f"blend {m}")


# ------------------------------------------------------------------ attention
def paged(k, v, page, seed, spare=3):
    """Keys [n, G, D] and values [n, G, V] in shuffled pages: pools and the one request's table."""
    n, G, D = k.shape
    V = v.shape[2]
    n_blocks = -(-n // page)
    order = torch.tensor(np.random.default_rng(seed).permutation(n_blocks + spare)[:n_blocks], dtype=torch.long)
    kpool = torch.full((n_blocks + spare, G, page, D), float("nan"), dtype=k.dtype)
    vpool = torch.full((n_blocks + spare, G, V, page), float("nan"), dtype=k.dtype)
    kp = torch.zeros(n_blocks * page, G, D, dtype=k.dtype)
    vp = torch.zeros(n_blocks * page, G, V, dtype=k.dtype)
    kp[:n], vp[:n] = k, v
    kpool[order] = kp.view(n_blocks, page, G, D).permute(0, 2, 1, 3)
    vpool[order] = vp.view(n_blocks, page, G, V).permute(0, 2, 3, 1)
    return kpool.to(DEV), vpool.to(DEV), order


def plain_attention(q, k, v, n_new, scale, window, cap, slopes, sink):
    """The last n_new rows of the plain attention over all n keys."""
    n, H = k.shape[0], q.shape[1]
    full_q = torch.zeros(n, H, q.shape[2], dtype=F)
    full_q[n - n_new:] = q.double()
    out = VP.attend(full_q, k.double(), v.double(), scale, window=window, cap=cap, slopes=None if slopes is None else slopes.double(),
                    sink=None if sink is None else sink.double())
    return out[n - n_new:]


def run_attention(kernel, dtype, q, k, v, n_new, scale, window, cap, slopes, sink, page, seed=0):
    """The last ``n_new`` positions of a request of len(k) tokens as one step through ``kernel``:
    "rows", "tiles" (prompt tiles on the matrix cores) or "split" (one new token, keys in partitions).
    Pages behind the window are given back first, as the cache manager does."""
    from lyapunov_engine_amd.kernels import ops
    from lyapunov_engine_amd.parts.attention import AttentionWork
    from lyapunov_engine_amd.parts.base import StepBatch

    n, G, D = k.shape
    H, V = q.shape[1], v.shape[2]
    first = n - n_new
    kpool, vpool, order = paged(k, v, page, seed)
    tb = order.numpy().astype(np.int32)[None, :].copy()
    if window:
        for b in range(max(0, first - window + 1) // page):
            kpool[tb[0, b]], vpool[tb[0, b]] = float("nan"), float("nan")
            tb[0, b] = -1
    table = ints(tb)
    qd = q.reshape(n_new, H * D).to(tdt(dtype)).to(DEV)
    out = torch.full((n_new, H * V), float("nan"), dtype=tdt(dtype), device=DEV)
    q_start, ctx_len, pos = ints([0, n_new]), ints([n]), ints(np.arange(first, n))
    f = lambda t: None if t is None else t.float().to(DEV)
    if kernel == "rows":
        ops.attn_rows(qd, out, kpool, vpool, table, q_start, pos, ctx_len, num_heads=H, num_kv_heads=G, dim=D, vdim=V,
                      scale=scale, window=window, sink=f(sink), cap=cap, slopes=f(slopes))
        return out.view(n_new, H, V)
    assert D == V
    batch = StepBatch(start=np.array([first], np.int32), count=np.array([n_new], np.int32),
                      q_start=np.array([0, n_new], np.int32), ctx_len=np.array([n], np.int32), T=n_new, B=1)
    arrays, meta = AttentionWork().plan(batch)
    common = dict(num_heads=H, num_kv_heads=G, head_dim=D, window=window, scale=scale, sink=f(sink), cap=cap, slopes=f(slopes))
    if kernel == "tiles":
        if n_new == 1:                                   # a lone token as a tile of its own
            arrays, meta = {"tile_seq": np.zeros(1, np.int32), "tile_q0": np.zeros(1, np.int32)}, dict(n_tiles=1)
        ops.attn_prefill(qd, out, kpool, vpool, table, q_start, ctx_len, ints(arrays["tile_seq"]), ints(arrays["tile_q0"]),
                         meta["n_tiles"], pair=False, **common)
    else:
        assert n_new == 1
        part = 256                                       # several partitions from 257 keys on
        max_parts = -(-n // part)
        part_o = torch.full((H * max_parts * D,), float("nan"), device=DEV)
        part_ml = torch.full((H * max_parts * 2,), float("nan"), device=DEV)
        ops.attn_decode(qd, out, kpool, vpool, table, q_start, ctx_len, None, 1, part_o, part_ml, max_parts, part, **common)
    return out.view(n_new, H, V)


CASES = [  # kernel, heads, kv heads, key size, value size, page
    ("rows", 3, 1, 10, 12, 4), ("rows", 2, 2, 32, 32, 16), ("rows", 4, 2, 24, 8, 8),
    ("tiles", 4, 2, 32, 32, 16), ("tiles", 2, 2, 16, 16, 4), ("tiles", 8, 1, 64, 64, 16), ("tiles", 3, 3, 48, 48, 8),
    ("tiles", 2, 1, 128, 128, 16),
]
SHAPES = [  # window, cap, slopes, sink
    (0, 0.0, False, None), (0, 4.0, False, "zero"), (44, 0.0, True, "learned"), (5, 3.0, True, None), (70, 50.0, False, "learned"),
    (0, 0.0, True, "zero"),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("shape", SHAPES)
def test_attention_over_pages(dtype, case, shape):
    """Random keys: whole prompts, a portion at the end of a long context, two tokens; a cap that
    bends most scores, slopes that differ from head to head, a learned sink and one of zero."""
    kernel, H, G, D, V, page = case
    window, cap, sloped, sink_kind = shape
    for n, n_new in ((37, 37), (150, 150), (333, 70), (333, 2)):
        g = torch.Generator().manual_seed(n + window)
        k = torch.randn(n, G, D, generator=g).to(tdt(dtype))
        v = torch.randn(n, G, V, generator=g).to(tdt(dtype))
        q = torch.randn(n_new, H, D, generator=g).to(tdt(dtype))
        sink = {None: None, "zero": torch.zeros(H), "learned": torch.randn(H, generator=g)}[sink_kind]
        slopes = VP.distance_slopes(H).float() * 4 if sloped else None
        scale = 2.5 * D ** -0.5
        want = plain_attention(q, k, v, n_new, scale, window, cap, slopes, sink)
        got = run_attention(kernel, dtype, q, k, v, n_new, scale, window, cap, slopes, sink, page, seed=n)
        close(got, want, dtype, f"{case} {shape}: {n_new} new of {n}", floor=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 32, 16), (2, 1, 64, 16), (3, 3, 16, 4), (16, 1, 16, 16), (2, 2, 128, 16)])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("n", [1, 5, 256, 257, 700, 1100])
def test_one_new_token_over_partitions(dtype, sizes, shape, n):
    H, G, D, page = sizes
    window, cap, sloped, sink_kind = shape
    g = torch.Generator().manual_seed(n + D)
    k = torch.randn(n, G, D, generator=g).to(tdt(dtype))
    v = torch.randn(n, G, D, generator=g).to(tdt(dtype))
    q = torch.randn(1, H, D, generator=g).to(tdt(dtype))
    sink = {None: None, "zero": torch.zeros(H), "learned": torch.randn(H, generator=g)}[sink_kind]
    slopes = VP.distance_slopes(H).float() * 0.2 if sloped else None
    scale = 2.5 * D ** -0.5
    want = plain_attention(q, k, v, 1, scale, window, cap, slopes, sink)
    got = run_attention("split", dtype, q, k, v, 1, scale, window, cap, slopes, sink, page, seed=n)
    close(got, want, dtype, f"{sizes} {shape}: one new token at {n - 1}", floor=0.1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kernel", ["rows", "tiles", "split"])
@pytest.mark.parametrize("window", [9, 44, 64, 130])
def test_a_planted_key_is_found_exactly_where_the_window_allows(dtype, kernel, window):
    """One key that the last query matches far better than any other, planted in turn at the
    window's two edges, page and tile edges, the first token and far back.  Where the window lets it
    be seen the output is its value (the cap is far above the score, the penalty small against it);
    elsewhere nothing of it may show."""
    H, G, D, page, n = 2, 1, 32, 16, 600
    pos = n - 1
    places = sorted({0, 15, 16, 255, 256, 300, pos - window - 1, pos - window, pos - window + 1, pos - window + 2, pos - 63,
                     pos - 64, pos - 1, pos} & set(range(n)))
    slopes = torch.tensor([0.01, 0.5])
    for where in places:
        g = torch.Generator().manual_seed(where)
        k = (torch.randn(n, G, D, generator=g) * 0.1).to(tdt(dtype))
        v = torch.randn(n, G, D, generator=g).to(tdt(dtype))
        q = torch.randn(1, H, D, generator=g)
        k[where, 0] = (q[0, 0] * 4).to(tdt(dtype))            # head 0 finds it; head 1 has its own random query
        q = q.to(tdt(dtype))
        seen = pos - where < window
        want = plain_attention(q, k, v, 1, 1.0, window, 500.0, slopes, torch.zeros(H))
        if seen:
            assert float((want[0, 0] - v[where, 0].double()).abs().max()) < 1e-2, "the case is meant to be decided by one key"
        got = run_attention(kernel, dtype, q, k, v, 1, 1.0, window, 500.0, slopes, torch.zeros(H), page, seed=where)
        close(got, want, dtype, f"{kernel} window {window}: a key planted at {where} ({'seen' if seen else 'not seen'})", floor=0.1)


@pytest.mark.parametrize("kernel", ["rows", "tiles", "split"])
def test_the_cap_bends_and_the_penalty_orders(kernel):
    """Two keys with equal large products: under a tight cap both scores are the cap and the
    penalty alone decides, the nearer key taking exp(slope * distance) times the weight."""
    dtype = "float32"
    H, G, D, page, n = 1, 1, 16, 16, 40
    k = torch.zeros(n, G, D)
    v = torch.zeros(n, G, D)
    q = torch.zeros(1, H, D)
    q[0, 0, 0] = 1.0
    k[:, 0, 0] = -50.0                       # everything else sits at minus the cap
    k[10, 0, 0] = k[30, 0, 0] = 50.0
    v[10, 0, 0], v[30, 0, 1] = 1.0, 1.0
    slopes = torch.tensor([0.1])
    got = run_attention(kernel, dtype, q, k, v, 1, 1.0, 0, 2.0, slopes, None, page)[0, 0].cpu()
    assert abs(float(got[1] / got[0]) - math.exp(0.1 * 20)) < 1e-3 * math.exp(2.0)
    want = plain_attention(q, k, v, 1, 1.0, 0, 2.0, slopes, None)
    close(got, want[0, 0], dtype, "cap and penalty")


# --------------------------------------------------- blends with the row before
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [8, 100, 192])
def test_blends_with_the_previous_row_over_steps_and_slots(dtype, C):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(C)
    mu = torch.rand(5, C, generator=g)
    state = torch.full((3, C), float("nan"), dtype=tdt(dtype), device=DEV)      # what a slot held before must not matter
    seqs = {0: torch.randn(9, C, generator=g).to(tdt(dtype)), 1: torch.randn(4, C, generator=g).to(tdt(dtype))}
    want = {r: torch.stack([VP.shifted(x.double()) * m + x.double() * (1 - m) for m in mu.double()]) for r, x in seqs.items()}
    done = {0: 0, 1: 0}
    slot = {0: 2, 1: 0}
    for step in ([(0, 3), (1, 1)], [(1, 2), (0, 1)], [(0, 5)], [(1, 1)]):
        rows = torch.cat([seqs[r][done[r]:done[r] + n] for r, n in step])
        starts = np.cumsum([0] + [n for _, n in step])
        pos = np.concatenate([np.arange(done[r], done[r] + n) for r, n in step])
        out = ops.shift_mix(rows.to(DEV), mu.to(DEV), state, ints(starts), ints(pos), ints([slot[r] for r, _ in step]), len(step))
        for i, (r, n) in enumerate(step):
            close(out[:, starts[i]:starts[i] + n], want[r][:, done[r]:done[r] + n], dtype, f"request {r} rows {done[r]}..")
            done[r] += n


# -------------------------------------------------------------- the recurrences
def plain_bonus_scan(r, k, v, decay, u, S=None):
    """o_t = (S + diag(u) k v^T)^T r;  S <- diag(decay) S + k v^T.  [T, H, d] each; S [H, d, dv]."""
    T, H, d = k.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F) if S is None else S.clone()
    o = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    return o, S


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(2, 48, 48), (1, 3, 5), (3, 64, 16), (2, 130, 8), (1, 300, 24), (4, 8, 64)])
def test_recurrence_with_a_bonus_for_the_current_token(dtype, sizes):
    """Portions down to one token, two requests side by side, a slot that another request left."""
    from lyapunov_engine_amd.kernels import ops

    H, d, dv = sizes
    g = torch.Generator().manual_seed(d)
    lens = {0: 45, 1: 7}
    data, want, S_end = {}, {}, {}
    for r, n in lens.items():
        rr, kk = torch.randn(n, H, d, generator=g).to(tdt(dtype)), (torch.randn(n, H, d, generator=g) * 0.5).to(tdt(dtype))
        vv = torch.randn(n, H, dv, generator=g).to(tdt(dtype))
        decay = torch.exp(-torch.exp(torch.randn(n, H, d, generator=g) - 1.0))
        data[r] = (rr, kk, vv, decay)
    u = torch.randn(H, d, generator=g)
    for r in lens:
        rr, kk, vv, decay = data[r]
        want[r], S_end[r] = plain_bonus_scan(rr.double(), kk.double(), vv.double(), decay.double(), u.double())
    state = torch.full((3, H, dv, d), 7.0, dtype=torch.float32, device=DEV)
    coef = torch.ones(H, device=DEV)
    done, slot = {0: 0, 1: 0}, {0: 1, 1: 2}
    for step in ([(0, 20)], [(0, 1), (1, 3)], [(1, 1), (0, 2)], [(0, 22), (1, 3)]):
        parts = [[data[r][i][done[r]:done[r] + n] for r, n in step] for i in range(4)]
        T = sum(n for _, n in step)
        rr, kk, vv = (torch.cat(p).reshape(T, -1).to(DEV) for p in parts[:3])
        decay = torch.cat(parts[3]).reshape(T, -1).float().to(DEV)
        starts = np.cumsum([0] + [n for _, n in step])
        pos = np.concatenate([np.arange(done[r], done[r] + n) for r, n in step])
        out = torch.empty(T, H * dv, device=DEV)
        ops.linear_scan(rr, kk, vv, decay, None, coef, 0.0, state, ints(starts), ints(pos), ints([slot[r] for r, _ in step]), out,
                        len(step), num_heads=H, num_kv_heads=H, dim=d, vdim=dv, bonus=u.reshape(-1).to(DEV))
        for i, (r, n) in enumerate(step):
            close(out[starts[i]:starts[i] + n].view(n, H, dv), want[r][done[r]:done[r] + n], dtype, f"request {r} from {done[r]}",
                  tol=3e-5 if dtype == "float32" else 3e-2)
            done[r] += n
    for r in lens:
        close(state[slot[r]].permute(0, 2, 1), S_end[r], "float32", f"the slot of request {r}", tol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 48, 32), (1, 1, 5, 3), (6, 1, 16, 16), (3, 3, 130, 8), (4, 2, 64, 64)])
def test_recurrence_with_one_decay_per_head_from_a_step_size(dtype, sizes):
    from lyapunov_engine_amd.kernels import ops

    H, G, N, dv = sizes
    g = torch.Generator().manual_seed(N)
    n = 41
    Bm, Cm = (torch.randn(n, G, N, generator=g) * 0.5).to(tdt(dtype)), torch.randn(n, G, N, generator=g).to(tdt(dtype))
    x = torch.randn(n, H, dv, generator=g).to(tdt(dtype))
    raw, bias, A = torch.randn(n, H, generator=g), torch.randn(H, generator=g), torch.exp(torch.randn(H, generator=g) * 0.7)
    dt = VP.softplus(raw.double() + bias.double())
    S = torch.zeros(H, N, dv, dtype=F)
    want = torch.zeros(n, H, dv, dtype=F)
    for t in range(n):
        for h in range(H):
            gg = h // (H // G)
            S[h] = torch.exp(-A[h].double() * dt[t, h]) * S[h] + dt[t, h] * Bm[t, gg].double()[:, None] * x[t, h].double()[None, :]
            want[t, h] = S[h].T @ Cm[t, gg].double()
    state = torch.full((2, H, dv, N), -3.0, dtype=torch.float32, device=DEV)
    at = 0
    for cut in (17, 1, 2, 21):
        sl = slice(at, at + cut)
        out = torch.empty(cut, H * dv, device=DEV)
        ops.linear_scan(Cm[sl].reshape(cut, -1).to(DEV), Bm[sl].reshape(cut, -1).to(DEV), x[sl].reshape(cut, -1).to(DEV),
                        raw[sl].to(DEV), bias.to(DEV), A.to(DEV), 1.0, state, ints([0, cut]), ints(np.arange(at, at + cut)), ints([1]),
                        out, 1, num_heads=H, num_kv_heads=G, dim=N, vdim=dv, z_per_head=True, key_step=True)
        close(out.view(cut, H, dv), want[sl], dtype, f"rows {at}..", tol=3e-5 if dtype == "float32" else 3e-2)
        at += cut
    close(state[1].permute(0, 2, 1), S, "float32", "the slot", tol=1e-4)


# ------------------------------------------------------------ row-wise kernels
@pytest.mark.parametrize("dtype", DTYPES)
def test_skip_gate_and_norm_in_groups(dtype):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(0)
    for T, H, V, groups in ((5, 4, 32, 2), (3, 3, 5, 3), (2, 6, 7, 1), (4, 8, 160, 4)):
        N = H * V
        o = torch.randn(T, N, generator=g)
        wide = torch.randn(T, 2 * N + 3, generator=g).to(tdt(dtype))       # z | x | more
        skip, w = torch.randn(H, generator=g), torch.randn(N, generator=g)
        got = ops.skip_gate_group_norm(o.to(DEV), wide[:, N:2 * N].to(DEV), skip.to(DEV), wide[:, :N].to(DEV), w.to(DEV), groups,
                                       1e-5, vdim=V)
        x, z = wide[:, N:2 * N].double(), wide[:, :N].double()
        y = (o.double() + skip.double().repeat_interleave(V) * x) * VP.silu(z)
        y = y.reshape(T, groups, N // groups)
        want = (y / VP.rms(y, 1e-5)).reshape(T, N) * w.double()
        close(got, want, dtype, f"{(T, H, V, groups)}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_gated_rows(dtype):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(1)
    table = torch.randn(50, 21, generator=g).to(tdt(dtype))
    p = torch.randn(7, 5, generator=g) * 2
    tok = torch.tensor([0, 49, 3, 3, 17, 20, 1], dtype=torch.int32)
    got = ops.gather_gelu_mul(p.to(DEV), tok.to(DEV), table.to(DEV)[:, 10:15])
    want = VP.gelu_tanh(p.double()) * table.double()[tok.long(), 10:15]
    close(got, want, dtype, "gelu(p) * row")


def test_decay_from_a_low_rank_pair_with_tanh_and_two_exponentials():
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(2)
    mid, w, b = torch.randn(11, 6, generator=g) * 2, torch.randn(40, 6, generator=g), torch.randn(40, generator=g)
    got = ops.lowrank_up(mid.to(DEV), w.to(DEV), b.to(DEV), mid_tanh=True, double_exp=True)
    want = torch.exp(-torch.exp(torch.tanh(mid.double()) @ w.double().T + b.double()))
    close(got, want, "float32", "exp(-exp(.))")


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_normed_with_weights_of_their_own(dtype):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(3)
    T, H, V = 6, 3, 20
    o, w = torch.randn(T, H * V, generator=g) * 3, torch.randn(H * V, generator=g)
    gate = torch.randn(T, H * V, generator=g).to(tdt(dtype))
    got = ops.head_norm_gate(o.to(DEV), w.to(DEV), gate.to(DEV), "silu", 1e-5, tdt(dtype), num_heads=H, vdim=V)
    oo = o.double().reshape(T, H, V)
    want = (oo / VP.rms(oo, 1e-5)).reshape(T, H * V) * w.double() * VP.silu(gate.double())
    close(got, want, dtype, "heads' norm")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_gate_per_head(dtype):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 3 * 7, generator=g).to(tdt(dtype))
    gate = torch.randn(5, 10, generator=g)
    got = ops.gate_mul(x.clone().to(DEV), gate.to(DEV)[:, 4:7], "sigmoid", per=7)
    want = x.double() * torch.sigmoid(gate.double()[:, 4:7]).repeat_interleave(7, dim=1)
    close(got, want, dtype, "one gate value a head")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [72, 192, 100])
def test_a_branch_joins_and_the_stream_is_copied_out(dtype, H):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(H)
    h, y, w = torch.randn(6, H, generator=g), torch.randn(6, H, generator=g).to(tdt(dtype)), torch.randn(H, generator=g)
    hd = h.clone().to(DEV)
    out = torch.empty(6, H, dtype=tdt(dtype), device=DEV)
    ops.branch_join(hd, y.to(DEV), (1 + w).to(DEV), 1.0, 1e-5, out=out)
    want = h.double() + VP.norm_one_plus(y.double(), w.double(), 1e-5)
    close(hd, want, "float32", "the stream")
    close(out, want, dtype, "its copy")
    rows = ints([4, 1])
    picked = torch.empty(2, H, dtype=tdt(dtype), device=DEV)
    before = hd.clone()
    ops.branch_join(hd, y.to(DEV), (1 + w).to(DEV), 1.0, 1e-5, out=picked, rows=rows)
    assert torch.equal(hd, before)
    close(picked, (want + VP.norm_one_plus(y.double(), w.double(), 1e-5))[[4, 1]], dtype, "picked rows")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C", [24, 7])
def test_convolution_with_a_bias(dtype, C):
    from lyapunov_engine_amd.kernels import ops

    g = torch.Generator().manual_seed(C)
    taps, n = 4, 12
    x = torch.randn(n, C + 5, generator=g).to(tdt(dtype))
    w, b = torch.randn(C, taps, generator=g) * 0.6, torch.randn(C, generator=g)
    want = VP.causal_conv(x[:, 2:2 + C].double(), w.double(), b.double())
    state = torch.full((2, taps - 1, C), float("nan"), dtype=tdt(dtype), device=DEV)
    at = 0
    for cut in (5, 1, 2, 4):
        out = torch.empty(cut, C, dtype=tdt(dtype), device=DEV)
        ops.short_conv(x[at:at + cut, 2:2 + C].to(DEV), w.to(DEV), state, ints([0, cut]), ints(np.arange(at, at + cut)), ints([1]), out, 1,
                       residual=False, silu=True, bias=b.to(DEV))
        close(out, want[at:at + cut], dtype, f"rows {at}..")
        at += cut
