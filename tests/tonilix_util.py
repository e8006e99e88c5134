"""Small Tonilix models with random weights for the tests, and their logits by
the plain implementation (tests/plain/tonilix_plain.py, 64-bit)."""
import json
import os

import torch

from plain import tonilix_plain as TP


def delta(heads, kv_heads, dim, vdim, conv, mlp=None):
    return dict(type="channel_delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv), mlp=mlp)


def pair(left, right, left_scale=1.0, right_scale=1.0, mlp=None):
    """left: (heads, kv_heads, dim, vdim, scale, coef, every); right: (heads, dim, vdim, tau)."""
    lh, lg, ld, lv, ls, coef, every = left
    rh, rd, rv, tau = right
    return dict(type="parallel", mlp=mlp, mixer=dict(
        left=dict(heads=lh, kv_heads=lg, dim=ld, vdim=lv, scale=ls, q_temp=dict(coef=coef, every=every)),
        right=dict(heads=rh, dim=rd, vdim=rv, tau=tau), left_scale=left_scale, right_scale=right_scale))


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, count, keep, scale):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale,
                                                            groups=dict(count=count, keep=keep)))


def config(vocab, width, layers, *, eps=1e-6, groups=1):
    return dict(architecture="Tonilix", vocab=vocab, width=width, norm=dict(eps=eps, groups=groups), layers=layers)


# Three configurations that differ in every size and option; none of their sizes coincide where a
# model's might by chance (key and value sizes, heads and key heads, heads x value size and width).
#   A: odd sizes (the row-by-row attention, the scalar paths), three norm groups, three taps, two key
#      heads for four heads in the recurrence, one key/value head for four query heads, a query
#      multiplier that changes every five positions, experts in three groups of which two are kept,
#      a layer without feed-forward
#   B: one of everything: one norm group, one tap (a convolution without memory), one head, a
#      multiplier from the first position on, as many groups as experts (groups of one) all kept,
#      one expert chosen, scales of 1
#   C: sizes in multiples of 16 (the matrix-core attention, the vector paths), keys of 128 values in
#      the recurrence (32 a lane), four taps, four norm groups, one of two groups kept
CONFIGS = {
    "A": config(203, 72, [pair((4, 1, 24, 20, 0.3, 0.7, 5), (3, 10, 12, 4.0), 0.8, 0.5, mlp=dense(100)),
                          delta(4, 2, 24, 10, 3, mlp=moe(6, 2, 40, 3, 2, 1.5)),
                          delta(2, 1, 12, 28, 3),
                          pair((2, 2, 12, 36, 0.25, 0.3, 16), (2, 20, 8, 9.0), 1.1, 0.7, mlp=moe(6, 3, 24, 3, 2, 2.5))],
                eps=1e-5, groups=3),
    "B": config(150, 64, [delta(1, 1, 32, 48, 1, mlp=moe(4, 1, 32, 4, 4, 1.0)),
                          pair((1, 1, 16, 16, 0.25, 1.0, 1), (1, 40, 24, 1.0), 1.0, 1.0, mlp=dense(48))],
                eps=1e-6, groups=1),
    "C": config(320, 128, [delta(2, 2, 128, 16, 4, mlp=dense(192)),
                           pair((4, 2, 32, 32, 0.18, 0.5, 32), (2, 64, 32, 16.0), 0.6, 0.9, mlp=moe(8, 3, 64, 2, 1, 2.0)),
                           delta(4, 1, 16, 32, 2, mlp=moe(8, 2, 48, 4, 3, 1.0))],
                eps=1e-6, groups=4),
}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 16}
# inner sizes of the low-rank pairs (decay, gate of the recurrence; decay of the linear attention): from the tensors alone
RANKS = {"A": (5, 7, 3), "B": (24, 8, 16), "C": (16, 32, 8)}


def write_model(folder: str, cfg: dict, seed: int, dtype: str, std: float = 0.2, ranks=(6, 4, 5)) -> str:
    """config.json and model.safetensors with weights drawn so that faults show: matrices wide
    enough for peaked attention and decays that differ from channel to channel, biases, corrections
    and shifts of order one half, scaling vectors and norm weights around one."""
    from lyapunov_engine_amd.config.registry import architecture_of
    from lyapunov_engine_amd.models.decoder import build_model
    from lyapunov_engine_amd.weights.safetensors_io import write_safetensors

    arch = architecture_of(cfg)
    model = build_model(arch.to_spec(arch.config_class.from_dict(cfg)))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, init) in model.expected_tensors().items():
        if any(d < 0 for d in shape):      # a low-rank pair's inner size: the file's to choose
            last = name.rsplit(".", 1)[-1]
            rank = ranks[2] if ".right." in name else (ranks[0] if last in ("a1", "a2") else ranks[1])
            shape = tuple(rank if d < 0 else d for d in shape)
        t = torch.randn(shape, generator=g)
        last = name.rsplit(".", 1)[-1]
        if init == "ones":
            t = 1.0 + 0.2 * t
        elif last in ("b",) and t.dim() == 1 or last in ("dt_bias",) or name.endswith("a2.b"):
            t = t * 1.0
        elif last == "correction":
            t = t * 0.3
        elif last == "shift":
            t = torch.sigmoid(t)
        elif last == "A_log":
            t = t * 0.7
        elif last == "conv":
            t = t * 0.6
        elif last == "router":
            t = t * 0.8
        elif name == "embed":
            t = t * 1.0
        elif last in ("a2", "g2"):
            t = t * (2.0 / shape[-1]) ** 0.5 * 2.0
        else:
            t = t * std * (32.0 / shape[-1]) ** 0.5
        tensors[name] = t.to(torch.bfloat16 if dtype == "bfloat16" else torch.float32)
    os.makedirs(folder, exist_ok=True)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return folder


_PLAIN: dict = {}


def _loaded(folder):
    if folder not in _PLAIN:
        _PLAIN[folder] = TP.load_folder(folder)
    return _PLAIN[folder]


def plain_logits(folder: str, requests: dict) -> dict:
    """id -> [len, vocab] 64-bit logits of every whole request."""
    cfg, tensors = _loaded(folder)
    return {rid: TP.forward(toks, tensors, cfg) for rid, toks in requests.items()}


class RouterLog:
    """Collects the engine's router choices while a trace is replayed (``with RouterLog() as log``)
    and sorts them by request: ``log.by_request(trace)`` -> id -> one tensor [len, top] per layer
    with a mixture of experts, in running order."""

    def __enter__(self):
        from lyapunov_engine_amd.parts.routed_experts import GroupRoutedExperts

        self.cls = GroupRoutedExperts
        self.cls.choices_log = self.calls = []
        return self

    def __exit__(self, *exc):
        self.cls.choices_log = None

    def by_request(self, trace) -> dict:
        steps = [s for s in trace.steps if s["entries"]]
        runs = len(self.calls) // max(1, len(steps))
        assert runs * len(steps) == len(self.calls)
        out = {rid: [[] for _ in range(runs)] for rid in trace.requests}
        for n, s in enumerate(steps):
            for r in range(runs):
                idx, at = self.calls[n * runs + r].cpu(), 0
                for e in s["entries"]:
                    out[e["id"]][r].append(idx[at:at + len(e["tokens"])])
                    at += len(e["tokens"])
        return {rid: [torch.cat(p) for p in per] if per and per[0] else [] for rid, per in out.items()}


def plain_logits_routed_alike(folder: str, requests: dict, chosen: dict, clear: float = 0.05) -> dict:
    """As ``plain_logits`` with the experts the engine chose.  A 16-bit run may decide a close call
    the other way, which says nothing about its kernels; what it must not do is choose otherwise
    where the plain model's margin is clear (more than ``clear``): that is asserted here."""
    cfg, tensors = _loaded(folder)
    out = {}
    for rid, toks in requests.items():
        out[rid] = TP.forward(toks, tensors, cfg, chosen=chosen[rid])
        notes = []
        TP.forward(toks, tensors, cfg, notes=notes)
        for run, (nf, theirs) in enumerate(zip(notes, chosen[rid])):
            differs = (torch.sort(theirs.long(), -1).values != torch.sort(nf["chosen"], -1).values).any(-1)
            if differs.any():
                first = int(torch.nonzero(differs)[0])      # later tokens follow another history
                assert float(nf["margin"][first]) < clear, (
                    f"request {rid!r}, routed layer {run}, position {first}: the engine chose {theirs[first].tolist()}, "
                    f"the plain model {nf['chosen'][first].tolist()} with a margin of {float(nf['margin'][first]):.3f}")
                break
    return out


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
