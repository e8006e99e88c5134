"""A plain, slow implementation of the Vobotar decoder in 64-bit torch on the
CPU, one function per mechanism, written from the design's equations and
sharing no code with the package.  Tensors come from a dict name -> tensor, the
configuration is the parsed config.json.

Notation: x is the residual stream [T, width]; a "head view" of a vector of
H * d values is [T, H, d]; positions count from 0.
"""
import json
import math
import os
import struct

import torch

F = torch.float64


# ------------------------------------------------------------------- reading
def read_safetensors(path):
    with open(path, "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        meta = json.loads(f.read(n))
        data = f.read()
    out = {}
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "I32": torch.int32, "F16": torch.float16}
    for name, e in meta.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        if hi == lo:
            out[name] = torch.zeros(e["shape"], dtype=kinds[e["dtype"]])
            continue
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[e["dtype"]])
        out[name] = t.reshape(e["shape"]).clone()
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    raw = read_safetensors(os.path.join(folder, "model.safetensors"))
    return cfg, {k: (v.to(F) if v.is_floating_point() else v) for k, v in raw.items()}


# ---------------------------------------------------------------- mechanisms
def rms(x, eps):
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """x / rms(x) * (1 + w): the weight is stored around zero."""
    return x / rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return x / rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def angles(positions, dims, base):
    """[T, dims / 2]: position * base^(-2i / dims)."""
    p = torch.as_tensor(positions, dtype=F)[:, None]
    i = torch.arange(dims // 2, dtype=F)[None, :]
    return p * torch.pow(torch.tensor(float(base), dtype=F), -2.0 * i / dims)


def rotate_neighbours(x, positions, dims, base):
    """x [T, H, d]: the pairs (2i, 2i + 1) of the first ``dims`` values of every head turn by the angle."""
    a = angles(positions, dims, base)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def rotate_halves(x, positions, dims, base):
    """x [T, H, d]: value i of the first ``dims`` is paired with value i + dims / 2."""
    a = angles(positions, dims, base)
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = x.clone()
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(T, window):
    """[T, T] bool: row i sees column j when j <= i and (no window or i - j < window)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def attend(q, k, v, scale, *, window=0, cap=0.0, slopes=None, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv].  Scores scale * q . k, capped by
    cap * tanh(s / cap) when cap > 0, less slopes[h] * (i - j) when there are slopes; softmax over the
    visible keys whose denominator also holds exp(sink[h]) when there is a sink (no value)."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    out = torch.zeros(T, H, v.shape[-1], dtype=F)
    ok = visible(T, window)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F)
    for h in range(H):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        if cap:
            s = cap * torch.tanh(s / cap)
        if slopes is not None:
            s = s - slopes[h] * dist
        s = s.masked_fill(~ok, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].reshape(1, 1).expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def distance_slopes(H):
    """2^(-8 (h + 1) / H) for head h."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=F)


def shifted(h, prev=None):
    """The previous token's row for every row (``prev`` or zeros for the first)."""
    first = torch.zeros_like(h[:1]) if prev is None else prev[None]
    return torch.cat([first, h[:-1]], 0)


def causal_conv(x, w, b, silu_after=True):
    """x [T, C], w [C, taps] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F), x], 0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    if b is not None:
        y = y + b
    return silu(y) if silu_after else y


# -------------------------------------------------------------------- mixers
def mixer_attention(h, positions, w, pre, m, eps, v_first):
    """Full causal attention: per-head normed q and k with a weight shared by the heads, neighbour
    rotation, capped scores, one more 1 in the softmax's denominator, values blended with the first
    such layer's, an element-wise sigmoid gate.  Returns (y, v as projected by this layer)."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + "q"].T).reshape(T, H, d)
    k = (h @ w[pre + "k"].T).reshape(T, G, d)
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    q = norm_plain(q, w[pre + "q.norm"], eps)
    k = norm_plain(k, w[pre + "k.norm"], eps)
    rot = m.get("rot")
    if rot:
        q = rotate_neighbours(q, positions, int(rot["dims"]), rot["base"])
        k = rotate_neighbours(k, positions, int(rot["dims"]), rot["base"])
    own_v = v
    if m.get("v_mix") and v_first is not None:
        lam = w[pre + "vmix"].reshape(())
        v = (1.0 - lam) * v + lam * v_first
    o = attend(q, k, v, float(m["scale"]), cap=float(m.get("softcap") or 0.0), sink=torch.zeros(H, dtype=F))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, own_v


def left_values_are_keys(h, positions, w, pre, m, eps):
    """Windowed attention whose values are the biased key projections; unit-rms q and k without a
    weight, no rotation, a distance penalty per head, a learned sink, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = k
    q = q / rms(q, eps)
    k = k / rms(k, eps)
    window = int(m["mask"]["size"]) if m.get("mask") else 0
    o = attend(q, k, v, float(m["scale"]), window=window, slopes=distance_slopes(H), sink=w[pre + "sink"])
    o = o * torch.sigmoid(h @ w[pre + "g"].T)[:, :, None]
    return o.reshape(T, -1) @ w[pre + "o"].T


def left_normed_projection(h, positions, w, pre, m, eps):
    """Windowed attention with biased q, k, v, one norm over each whole q and k projection, rotation of
    halves, a plain softmax, a sigmoid gate per head."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ w[pre + "q"].T + w[pre + "q.b"]
    k = h @ w[pre + "k"].T + w[pre + "k.b"]
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, dv)
    q = norm_plain(q, w[pre + "q.norm"], eps).reshape(T, H, d)
    k = norm_plain(k, w[pre + "k.norm"], eps).reshape(T, G, d)
    rot = m.get("rot")
    if rot:
        q = rotate_halves(q, positions, int(rot["dims"]), rot["base"])
        k = rotate_halves(k, positions, int(rot["dims"]), rot["base"])
    window = int(m["mask"]["size"]) if m.get("mask") else 0
    o = attend(q, k, v, float(m["scale"]), window=window)
    o = o * torch.sigmoid(h @ w[pre + "g"].T)[:, :, None]
    return o.reshape(T, -1) @ w[pre + "o"].T


def right_time_mix(h, w, pre, m, eps, state=None):
    """A matrix per head with a decay per key channel and a bonus for the current token.  ``state``:
    (S [H, d, d], the previous token's h) or None for a sequence's start; returns (y, state)."""
    T = h.shape[0]
    H, d = int(m["heads"]), int(m["dim"])
    S, prev = (torch.zeros(H, d, d, dtype=F), None) if state is None else (state[0].clone(), state[1])
    before = shifted(h, prev)
    mix = {s: h + (before - h) * w[pre + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ w[pre + "r"].T).reshape(T, H, d)
    k = (mix["k"] @ w[pre + "k"].T).reshape(T, H, d)
    v = (mix["v"] @ w[pre + "v"].T).reshape(T, H, d)
    gate = silu(mix["g"] @ w[pre + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"])).reshape(T, H, d)
    u = w[pre + "u"].reshape(H, d)
    o = torch.zeros(T, H, d, dtype=F)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]                       # [H, d, d]
        o[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    o = o / rms(o, eps)
    y = (o.reshape(T, H * d) * w[pre + "norm"] * gate) @ w[pre + "o"].T
    return y, (S, h[-1].clone())


def right_state_space(h, w, pre, m, eps, state=None):
    """A state-space layer with a scalar decay per head.  ``state``: (S [H, N, dv], the convolution's
    last taps - 1 inputs [taps - 1, channels]) or None; returns (y, state)."""
    T = h.shape[0]
    H, dv, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    taps, parts = int(m["conv"]), int(m["norm_groups"])
    inner = H * dv
    p = h @ w[pre + "in"].T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    C = xbc.shape[1]
    S, tail = (torch.zeros(H, N, dv, dtype=F), torch.zeros(taps - 1, C, dtype=F)) if state is None else (state[0].clone(), state[1])
    wc, bc = w[pre + "conv"], w.get(pre + "conv.b")
    seq = torch.cat([tail, xbc], 0)
    act = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        act = act + seq[j:j + T] * wc[:, j]
    if bc is not None:
        act = act + bc
    act = silu(act)
    new_tail = seq[seq.shape[0] - (taps - 1):].clone() if taps > 1 else tail
    xs = act[:, :inner].reshape(T, H, dv)
    Bm = act[:, inner:inner + G * N].reshape(T, G, N)
    Cm = act[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])
    A = torch.exp(w[pre + "A_log"])
    y = torch.zeros(T, H, dv, dtype=F)
    rep = H // G
    for t in range(T):
        for hd in range(H):
            g = hd // rep
            S[hd] = torch.exp(-A[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * Bm[t, g][:, None] * xs[t, hd][None, :]
            y[t, hd] = S[hd].T @ Cm[t, g] + w[pre + "D"][hd] * xs[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = y.reshape(T, parts, inner // parts)
    y = (y / rms(y, eps)).reshape(T, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T, (S, new_tail)


def feed_forward(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def token_side(x, tokens, w, layer, dim, eps):
    """What a layer adds from the token itself: the layer's stretch of the token's side row gates a
    small projection of x; the result is rms-normed with a plain weight."""
    e = w["side.embed"][torch.as_tensor(tokens, dtype=torch.long)][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return norm_plain(y, w[f"l{layer}.side.norm"], eps)


# --------------------------------------------------------------------- model
def forward(cfg, w, tokens, return_layers=False, positions=None):
    """Logits [T, vocab] for one whole sequence from position 0."""
    T = len(tokens)
    pos = list(range(T)) if positions is None else positions
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    side = cfg.get("token_side")
    v_first = None
    layers = []
    for i, lc in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", lc["mixer"]
        if lc["type"] == "attention":
            y, own_v = mixer_attention(x, pos, w, pre, m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = own_v
        elif lc["type"] == "parallel":
            a = left_values_are_keys(x, pos, w, pre + "left.", m["left"], eps)
            b, _ = right_time_mix(x, w, pre + "right.", m["right"], eps)
            y = float(m["left_scale"]) * a + float(m["right_scale"]) * b
        elif lc["type"] == "parallel_2":
            a = left_normed_projection(x, pos, w, pre + "left.", m["left"], eps)
            b, _ = right_state_space(x, w, pre + "right.", m["right"], eps)
            y = float(m["left_scale"]) * a + float(m["right_scale"]) * b
        else:
            raise ValueError(lc["type"])
        x = x + norm_one_plus(y, w[f"l{i}.norm1"], eps)
        if lc.get("mlp") is not None:
            x = x + norm_one_plus(feed_forward(x, w, f"l{i}.mlp."), w[f"l{i}.norm2"], eps)
        if side:
            x = x + token_side(x, tokens, w, i, int(side["dim"]), eps)
        layers.append(x.clone())
    logits = norm_one_plus(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, torch.stack(layers)) if return_layers else logits
