"""Small Vobotar models with random weights for the tests, and their logits by
the plain implementation (tests/plain/vobotar_plain.py, 64-bit)."""
import json
import os

import torch

from plain import vobotar_plain as VP


def dense(ff):
    return dict(kind="dense", ff=ff)


def attention(heads, kv_heads, dim, vdim, scale, rot=None, softcap=None, v_mix=False, mlp=None):
    """rot: (base, dims) or None."""
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot is not None:
        m["rot"] = dict(base=rot[0], dims=rot[1])
    if softcap is not None:
        m["softcap"] = softcap
    if v_mix:
        m["v_mix"] = True
    return dict(type="attention", mixer=m, mlp=mlp)


def _left(heads, kv_heads, dim, vdim, scale, window=None, rot=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if window:
        m["mask"] = dict(size=window)
    if rot is not None:
        m["rot"] = dict(base=rot[0], dims=rot[1])
    return m


def pair(left, right, left_scale=1.0, right_scale=1.0, mlp=None):
    """Attention whose values are its keys beside a time mix.  left: (heads, kv_heads, dim, scale,
    window or None); right: (heads, dim)."""
    h, g, d, s, win = left
    return dict(type="parallel", mlp=mlp, mixer=dict(left=_left(h, g, d, d, s, win), right=dict(heads=right[0], dim=right[1]),
                                                     left_scale=left_scale, right_scale=right_scale))


def pair2(left, right, left_scale=1.0, right_scale=1.0, mlp=None):
    """Attention with normed projections beside a state-space layer.  left: (heads, kv_heads, dim,
    vdim, scale, window or None, rot or None); right: (heads, vdim, state, groups, conv, norm_groups)."""
    h, g, d, dv, s, win, rot = left
    rh, rv, n, rg, taps, ng = right
    return dict(type="parallel_2", mlp=mlp, mixer=dict(
        left=_left(h, g, d, dv, s, win, rot), right=dict(heads=rh, vdim=rv, state=n, groups=rg, conv=taps, norm_groups=ng),
        left_scale=left_scale, right_scale=right_scale))


def config(vocab, width, layers, *, eps=1e-6, scale=1.0, side=0):
    d = dict(architecture="Vobotar", vocab=vocab, width=width, embedding=dict(scale=scale), norm=dict(eps=eps), layers=layers)
    if side:
        d["token_side"] = dict(dim=side)
    return d


def random_config(rng) -> dict:
    """A configuration drawn at random: width, vocabulary, one to six layers of any kind in any
    order, heads and key/value heads, key and value sizes that are equal or not (the matrix-core
    kernels or the row-by-row one), windows from one token up, rotations of two values up to the
    whole head, caps, blended values, taps, groups, with and without feed-forward and side input."""
    def divisors(n):
        return [d for d in range(1, n + 1) if n % d == 0]

    width = rng.choice([48, 64, 96, 128, 160, 192, 256])
    sizes = [8, 16, 24, 32, 48, 64, 80, 96, 128]
    g_att, vd_att = rng.choice([1, 2, 4]), rng.choice([8, 16, 32, 48, 64])     # blending layers share the values' shape
    layers = []
    for _ in range(rng.randint(1, 6)):
        kind = rng.choice(["attention", "parallel", "parallel_2"])
        mlp = None if rng.random() < 0.2 else dense(rng.choice([32, 64, 100, 192, 320]))
        scale = lambda d: round(d ** -0.5 * rng.uniform(0.7, 2.0), 4)
        if kind == "attention":
            d = vd_att if rng.random() < 0.4 else rng.choice(sizes)
            rot = None if rng.random() < 0.2 else (rng.choice([100.0, 1e4, 1e6]), rng.choice(range(2, d + 1, 2)))
            layers.append(attention(g_att * rng.choice([1, 2, 3, 4]), g_att, d, vd_att, scale(d), rot=rot,
                                    softcap=rng.choice([None, 5.0, 20.0, 50.0]), v_mix=rng.random() < 0.7, mlp=mlp))
        elif kind == "parallel":
            g, d = rng.choice([1, 2, 4, 8]), rng.choice(sizes[:8])
            layers.append(pair((g * rng.choice([1, 2, 3]), g, d, scale(d), rng.choice([None, 1, 7, 16, 33, 72, 150])),
                               (rng.choice([1, 2, 3, 4]), rng.choice([8, 16, 24, 48, 64, 100])),
                               round(rng.uniform(0.3, 1.5), 2), round(rng.uniform(0.3, 1.5), 2), mlp=mlp))
        else:
            g, d = rng.choice([1, 2, 4]), rng.choice(sizes)
            dv = d if rng.random() < 0.6 else rng.choice(sizes)
            rot = None if rng.random() < 0.2 else (rng.choice([100.0, 2.5e5]), rng.choice(range(2, d + 1, 2)))
            heads = rng.choice([1, 2, 4, 6])
            layers.append(pair2((g * rng.choice([1, 2, 3]), g, d, dv, scale(d), rng.choice([None, 2, 9, 31, 64, 136]), rot),
                                (heads, rng.choice([8, 16, 32]), rng.choice([8, 16, 48, 64, 100]), rng.choice(divisors(heads)),
                                 rng.choice([1, 2, 3, 4, 5]), rng.choice(divisors(heads))),
                                round(rng.uniform(0.3, 1.5), 2), round(rng.uniform(0.3, 1.5), 2), mlp=mlp))
    return config(rng.randint(100, 600), width, layers, eps=rng.choice([1e-6, 1e-5]), scale=rng.choice([0.5, 1.0, 2.0]),
                  side=rng.choice([0, 4, 12, 16, 32]))


# Three configurations that differ in every size and option; none of their sizes coincide where a
# model's might by chance (key and value sizes, heads and key heads, heads x value size and width).
#   A: odd sizes (the row-by-row attention, the scalar paths): keys of 10 with values of 12, one
#      key/value head for three query heads, six rotated values of ten, windows shorter than a page
#      and no multiple of it, three taps, one group for three state-space heads, three norm groups,
#      a layer without feed-forward, blended values in the second and third attention layer
#   B: one of everything: one head everywhere, one tap (a convolution without memory), one norm
#      group, no token side input, no rotation, no cap, no blending, no window on one pair
#   C: sizes in multiples of 16 (the matrix-core attention with cap, slopes and sinks; the vector
#      paths): heads of 32 and 64, recurrence keys of 128, four taps, windows of several pages
CONFIGS = {
    "A": config(203, 72, [
        attention(3, 1, 10, 12, 0.4, rot=(300.0, 6), softcap=5.0, v_mix=True, mlp=dense(100)),
        pair((4, 2, 14, 0.35, 21), (3, 10), 0.8, 0.5, mlp=dense(60)),
        attention(2, 1, 8, 12, 0.5, rot=(5000.0, 8), softcap=9.0, v_mix=True),
        pair2((6, 2, 6, 10, 0.45, 13, (700.0, 4)), (3, 8, 12, 1, 3, 3), 1.1, 0.7, mlp=dense(44)),
        attention(4, 1, 6, 12, 0.3, softcap=30.0, v_mix=True, mlp=dense(36)),
    ], eps=1e-5, scale=0.7, side=5),
    "B": config(150, 64, [
        pair2((1, 1, 24, 8, 0.3, None, None), (1, 40, 24, 1, 1, 1), 1.0, 1.0, mlp=dense(48)),
        attention(1, 1, 16, 24, 0.25),
        pair((1, 1, 40, 0.2, None), (1, 24), 1.0, 1.0, mlp=dense(40)),
    ], eps=1e-6, scale=1.0),
    "C": config(320, 128, [
        pair((4, 2, 32, 0.18, 40), (2, 128), 0.6, 0.9, mlp=dense(192)),
        attention(4, 2, 64, 64, 0.12, rot=(1e5, 32), softcap=12.0, v_mix=True, mlp=dense(160)),
        pair2((4, 4, 32, 32, 0.2, 72, (1e4, 32)), (4, 16, 64, 2, 4, 2), 0.5, 1.5, mlp=dense(96)),
        attention(2, 2, 64, 64, 0.15, rot=(1e6, 64), softcap=20.0, v_mix=True, mlp=dense(64)),
    ], eps=1e-6, scale=0.5, side=16),
}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 16}
RANKS = {"A": 5, "B": 24, "C": 16}     # inner size of the decay's low-rank pair: from the tensors alone


def write_model(folder: str, cfg: dict, seed: int, dtype: str, std: float = 0.25, rank: int = 6) -> str:
    """config.json and model.safetensors with weights drawn so that faults show: projections wide
    enough for peaked attention, biases and sinks of order one, decays that differ from channel to
    channel and from head to head, blends away from 0 and 1, norm weights away from their rest value."""
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors

    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, init) in model.expected_tensors().items():
        shape = tuple(rank if d < 0 else d for d in shape)
        t = torch.randn(shape, generator=g)
        last = name.rsplit(".", 1)[-1]
        if init == "ones":                                   # plain norm weights, the state space's skip
            t = 1.0 + 0.3 * t
        elif last in ("norm1", "norm2") or name == "final.norm":
            t = 0.3 * t                                      # stored around zero
        elif last == "b" and t.dim() == 1:
            t = t * (0.3 if name.endswith("conv.b") else 0.7)
        elif last in ("r", "k", "v", "g") and ".mu." in name or last == "w" and ".mu." in name:
            t = torch.sigmoid(t)
        elif last == "vmix":
            t = torch.sigmoid(t) * 0.8 + 0.1
        elif last == "sink":
            t = t * 1.5
        elif last == "u":
            t = t * 0.6
        elif last == "w0":
            t = t * 0.8 - 1.0
        elif last in ("A_log", "dt_bias"):
            t = t * 0.7
        elif last == "conv":
            t = t * 0.6
        elif last == "w2":
            t = t * (2.0 / shape[-1]) ** 0.5 * 1.5
        elif name in ("embed", "side.embed"):
            t = t * 1.0
        elif name.endswith(".side.gate"):
            # what gates the token's row stays of order one: far below zero gelu gives nothing, and a branch
            # that is nearly nothing has its rounding blown up by the norm that follows it
            t = t * 0.4 / shape[-1] ** 0.5
        else:
            t = t * std * (32.0 / shape[-1]) ** 0.5
        tensors[name] = t.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    for name in model.spec.ignorable_tensors:                # what a file holds although nothing reads it
        if name.endswith("vmix"):
            tensors[name] = torch.tensor(0.5).to(torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


_PLAIN: dict = {}


def _loaded(folder):
    if folder not in _PLAIN:
        _PLAIN[folder] = VP.load_folder(folder)
    return _PLAIN[folder]


def forget(folder):
    _PLAIN.pop(folder, None)


def plain_logits(folder: str, requests: dict) -> dict:
    """id -> [len, vocab] 64-bit logits of every whole request."""
    cfg, tensors = _loaded(folder)
    return {rid: VP.forward(cfg, tensors, toks) for rid, toks in requests.items()}


def plain_sensitivity(folder: str, requests: dict, rel: float = 2.0 ** -9, seed: int = 0) -> dict:
    """id -> [len]: by how much a row's logits move when every matrix entry is changed by up to one
    rounding step of a 16-bit number (a relative ``rel``, drawn at random).  Every branch of this
    design is divided by its own root mean square, some parts of it by the root mean square of a
    few values; a row in which such a divisor happens to be small carries its rounding many times
    enlarged, and this is the measure of it."""
    cfg, tensors = _loaded(folder)
    g = torch.Generator().manual_seed(seed)
    moved = {k: v * (1.0 + rel * (2.0 * torch.rand(v.shape, generator=g, dtype=v.dtype) - 1.0))
             if v.is_floating_point() and v.dim() >= 2 else v for k, v in tensors.items()}
    return {rid: (VP.forward(cfg, moved, toks) - VP.forward(cfg, tensors, toks)).abs().max(-1).values
            for rid, toks in requests.items()}


def plain_greedy(folder: str, prompt: list, n: int):
    """n greedy tokens after the prompt, and the margin between the best two logits at each."""
    toks, out, margins = list(prompt), [], []
    for _ in range(n):
        row = plain_logits(folder, {"g": toks})["g"][-1]
        top = torch.topk(row, 2)
        out.append(int(top.indices[0]))
        margins.append(float(top.values[0] - top.values[1]))
        toks.append(out[-1])
    return out, margins


def edit(folder, change):
    """Rewrite a written model's tensors: ``change(tensors)`` edits the dict name -> tensor in place."""
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors

    path = os.path.join(folder, "model.safetensors")
    tensors = dict(VP.read_safetensors(path))
    change(tensors)
    write_safetensors(path, tensors, metadata={"format": "pt"})
    forget(folder)
