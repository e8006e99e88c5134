"""A plain, slow implementation of the Tonilix decoder in 64-bit torch on the
CPU, one function per mechanism, written from the design's equations and
sharing no code with the package.  Tensors come from a dict name -> tensor, the
configuration is the parsed config.json.

Notation: x is the residual stream [T, width]; a "head view" of a vector of
H * d values is [T, H, d].
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
    for name, e in meta.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = bytearray(data[lo:hi])
        if e["dtype"] == "BF16":
            t = torch.frombuffer(raw, dtype=torch.bfloat16)
        elif e["dtype"] == "F32":
            t = torch.frombuffer(raw, dtype=torch.float32)
        elif e["dtype"] == "I32":
            t = torch.frombuffer(raw, dtype=torch.int32)
        else:
            raise ValueError(f"{name}: dtype {e['dtype']}")
        out[name] = t.reshape(e["shape"]).clone()
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {k: (v.to(F) if v.is_floating_point() else v) for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


# ---------------------------------------------------------------- mechanisms
def sinusoid(positions, width):
    """[T, width]: entry 2i is sin(p * 10000^(-2i / width)), entry 2i + 1 the cosine of the same angle."""
    p = torch.as_tensor(positions, dtype=F)[:, None]
    i = torch.arange((width + 1) // 2, dtype=F)[None, :]
    ang = p * torch.pow(torch.tensor(10000.0, dtype=F), -2.0 * i / width)
    out = torch.zeros(p.shape[0], 2 * i.shape[1], dtype=F)
    out[:, 0::2] = torch.sin(ang)
    out[:, 1::2] = torch.cos(ang)
    return out[:, :width]


def group_rms_norm(x, w, eps, groups):
    """Every one of ``groups`` equal consecutive parts of a row divided by its own root mean square
    (eps inside the root); the whole row times w."""
    T, C = x.shape
    g = x.reshape(T, groups, C // groups)
    g = g / torch.sqrt((g * g).mean(-1, keepdim=True) + eps)
    return g.reshape(T, C) * w


def token_shift(n, mu, prev=None):
    """n_t + (n_(t-1) - n_t) * mu with n_(-1) = prev (zeros at a sequence's start)."""
    before = torch.cat([torch.zeros_like(n[:1]) if prev is None else prev[None], n[:-1]], 0)
    return n + (before - n) * mu


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def causal_conv(x, w, before=None):
    """x [T, C], w [C, taps] (last column: the current token): y_t = sum_j w[:, j] x_(t - taps + 1 + j),
    zeros (or ``before``, the taps - 1 inputs that came earlier) in front."""
    taps = w.shape[1]
    pad = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype) if before is None else before
    xx = torch.cat([pad, x], 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + xx[j:j + x.shape[0]] * w[:, j]
    return y


def head_rms_gate(o, w, eps, gate):
    """o [T, H, d]: every head over its d values divided by its root mean square, times w [d], times gate [T, H, d]."""
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
    return o * w * gate


def delta_rule_scan(q, k, v, g, beta, S=None):
    """Per head, token by token:  S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t.
    q, k, g [T, H, d]; v [T, H, e]; beta [T, H]; S [H, d, e].  Returns (o [T, H, e], S)."""
    T, H, d = q.shape
    e = v.shape[-1]
    S = torch.zeros(H, d, e, dtype=F) if S is None else S.clone()
    o = torch.zeros(T, H, e, dtype=F)
    for t in range(T):
        S = S * g[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + torch.einsum("hd,he->hde", k[t], u)
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    return o, S


def decayed_outer_scan(q, k, v, a, S=None):
    """Per head:  S_t = diag(a_t) S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t."""
    T, H, d = q.shape
    e = v.shape[-1]
    S = torch.zeros(H, d, e, dtype=F) if S is None else S.clone()
    o = torch.zeros(T, H, e, dtype=F)
    for t in range(T):
        S = S * a[t][:, :, None] + torch.einsum("hd,he->hde", k[t], v[t])
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    return o, S


def channel_delta(h, w, pre, m, eps):
    """The gated-delta mixer on a whole sequence h [T, width]."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(T, G, d)
    k = silu(causal_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(T, G, d)
    v = silu(causal_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(T, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]
    g = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * softplus(z).reshape(T, H, d))
    o, _ = delta_rule_scan(q, k, v, g, beta)
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).reshape(T, H, e)
    return head_rms_gate(o, w[pre + "norm"], eps, gate).reshape(T, H * e) @ w[pre + "o"].T


def tempered_attention(h, w, pre, m, positions):
    """Softmax attention with biases, a query multiplier that grows with the position, and a sigmoid output gate."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, e)
    p = torch.as_tensor(positions, dtype=torch.int64)
    temp = 1.0 + m["q_temp"]["coef"] * torch.log(torch.div(p + 1, m["q_temp"]["every"], rounding_mode="floor").to(F) + 1.0)
    q = q * temp[:, None, None]
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    s = torch.einsum("thd,jhd->htj", q, k) * m["scale"]
    s = s.masked_fill(p[None, None, :] > p[None, :, None], float("-inf"))
    o = torch.einsum("htj,jhe->the", torch.softmax(s, -1), v).reshape(T, H * e)
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T + w[pre + "o.b"]


def gated_linear_attention(h, w, pre, m, eps):
    T = h.shape[0]
    H, d, e = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, d)
    v = (h @ w[pre + "v"].T).reshape(T, H, e)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    a = torch.pow(torch.sigmoid(z), 1.0 / m["tau"]).reshape(T, H, d)
    o, _ = decayed_outer_scan(q, k, v, a)
    gate = silu(h @ w[pre + "g"].T).reshape(T, H, e)
    return head_rms_gate(o, w[pre + "norm"], eps, gate).reshape(T, H * e) @ w[pre + "o"].T


def side_by_side(h, w, pre, m, eps, positions):
    left = tempered_attention(h, w, pre + "left.", m["left"], positions)
    right = gated_linear_attention(h, w, pre + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def gated_dense(h, w, pre):
    return (gelu_tanh(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def choose_experts(s, correction, r, margin_out=None):
    """s [T, E] sigmoid scores -> (chosen [T, top] indices, weights [T, top]).  Experts are chosen by
    s + correction among the ``keep`` groups (of ``count`` groups of neighbours) whose two largest
    choice scores add up highest; the weights are the chosen experts' plain s over their sum, times r.scale.
    ``margin_out``: a list that receives, per token, how clear the choice was (the smaller of the gap
    between the last kept and the first dropped group and the gap between the last chosen and the
    first not chosen expert)."""
    T, E = s.shape
    c = s + correction
    count, keep = r["groups"]["count"], r["groups"]["keep"]
    per = E // count
    grouped = c.reshape(T, count, per)
    gscore = torch.topk(grouped, min(2, per), -1).values.sum(-1)
    gsorted = torch.sort(gscore, -1, descending=True).values
    kept = torch.topk(gscore, keep, -1).indices
    allowed = torch.zeros(T, count, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    c = c.masked_fill(~allowed[:, :, None].expand(T, count, per).reshape(T, E), float("-inf"))
    csorted = torch.sort(c, -1, descending=True).values
    chosen = torch.topk(c, r["top"], -1).indices
    if margin_out is not None:
        big = torch.full((T,), float("inf"), dtype=s.dtype)
        g_gap = gsorted[:, keep - 1] - gsorted[:, keep] if keep < count else big
        e_gap = csorted[:, r["top"] - 1] - csorted[:, r["top"]] if r["top"] < keep * per else big
        margin_out.append(torch.minimum(g_gap, e_gap))
    return chosen, route_weights(s, chosen, r)


def route_weights(s, chosen, r):
    ws = torch.gather(s, 1, chosen)
    return ws / (ws.sum(-1, keepdim=True) + 1e-20) * r["scale"]


def expert_mixture(h, w, pre, mlp, chosen=None, note=None):
    """``chosen`` [T, top]: experts to use instead of the router's own choice (the weights still come
    from the scores); ``note``: a dict that receives the own choice and its margins."""
    r = mlp["router"]
    s = torch.sigmoid(h @ w[pre + "router"].T)
    margins = []
    own, weights = choose_experts(s, w[pre + "correction"], r, margins)
    if note is not None:
        note.update(chosen=own, margin=margins[0])
    if chosen is not None:
        own, weights = chosen.long(), route_weights(s, chosen.long(), r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, e in enumerate(own[t].tolist()):
            a = torch.relu(h[t] @ w[f"{pre}e{e}.up"].T) ** 2
            out[t] += weights[t, j] * (a @ w[f"{pre}e{e}.down"].T)
    return out


# ------------------------------------------------------------------ the model
def forward(tokens, w, cfg, layers_out=None, chosen=None, notes=None):
    """float64 logits [T, vocab] of one whole sequence; ``layers_out``: a list that receives the
    residual stream after every layer; ``chosen``: one tensor [T, top] per layer with a mixture of
    experts, in order, to be used instead of the routers' own choices; ``notes``: a list that
    receives a dict (own choice, margins) per such layer."""
    moe_at = 0
    T, C = len(tokens), cfg["width"]
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    positions = list(range(T))
    norm = lambda x, name: group_rms_norm(x, w[name], eps, groups)
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.int64)] + sinusoid(positions, C)
    x = norm(x, "embed.norm")
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = token_shift(norm(x, p + "norm1"), w[p + "shift"])
        if layer["type"] == "channel_delta":
            y = channel_delta(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = side_by_side(h, w, p + "mix.", layer["mixer"], eps, positions)
        else:
            raise ValueError(layer["type"])
        x = x + y * w[p + "ls1"]
        if layer.get("mlp") is not None:
            h = norm(x, p + "norm2")
            if layer["mlp"]["kind"] == "dense":
                y = gated_dense(h, w, p + "mlp.")
            else:
                note = {} if notes is not None else None
                y = expert_mixture(h, w, p + "mlp.", layer["mlp"], None if chosen is None else chosen[moe_at], note)
                moe_at += 1
                if notes is not None:
                    notes.append(note)
            x = x + y * w[p + "ls2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm(x, "final.norm") @ w["head"].T


def greedy(logits_row):
    return int(torch.argmax(logits_row))
