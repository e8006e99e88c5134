"""Typed configuration of the Vobotar decoder, read from config.json.

The file names its architecture in the singular (``"architecture": "Vobotar"``)
and nests its constants: ``vocab``, ``width``, ``embedding`` (``scale``), ``norm``
(``eps``), ``token_side`` (``dim``; absent: layers take nothing from the token
itself) and ``layers``, a list whose entries give ``type`` (which mixer),
``mixer`` (its sizes and constants) and ``mlp`` (its feed-forward, or null):

    type "attention"    mixer: heads, kv_heads, dim, vdim, scale; optional rot {base, dims}, softcap, v_mix
    type "parallel"     mixer: left {heads, kv_heads, dim, vdim, scale; optional mask {size}},
                               right {heads, dim}, left_scale, right_scale
    type "parallel_2"   mixer: left {heads, kv_heads, dim, vdim, scale; optional mask {size}, rot {base, dims}},
                               right {heads, vdim, state, groups, conv, norm_groups}, left_scale, right_scale
    mlp kind "dense"    ff

Every size and constant comes from the file (the inner size of a low-rank
projection from the tensors' shapes); a missing one is an error that names it.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

from .model_config import ConfigError

MIXER_TYPES = ("attention", "parallel", "parallel_2")
MLP_KINDS = ("dense",)


def _need(d, keys, where: str) -> None:
    if not isinstance(d, dict):
        raise ConfigError(f"{where} must be an object, got {type(d).__name__}")
    missing = [k for k in keys if k not in d]
    if missing:
        raise ConfigError(f"{where} lacks {missing}")


def _positive(d: dict, keys, where: str) -> None:
    for k in keys:
        if not float(d[k]) > 0:
            raise ConfigError(f"{where}.{k} must be positive, got {d[k]}")


def _attention(m: dict, where: str) -> None:
    _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where)
    _positive(m, ("heads", "kv_heads", "dim", "vdim"), where)
    if int(m["heads"]) % int(m["kv_heads"]):
        raise ConfigError(f"{where}: {m['heads']} query heads do not split over {m['kv_heads']} key/value heads")
    if m.get("rot") is not None:
        _need(m["rot"], ("base", "dims"), where + ".rot")
        dims = int(m["rot"]["dims"])
        if dims < 0 or dims % 2 or dims > int(m["dim"]) or not float(m["rot"]["base"]) > 0:
            raise ConfigError(f"{where}.rot: {dims} rotated values of {m['dim']}, base {m['rot']['base']}")
    if m.get("mask") is not None:
        _need(m["mask"], ("size",), where + ".mask")
        if int(m["mask"]["size"]) < 1:
            raise ConfigError(f"{where}.mask.size must be at least 1, got {m['mask']['size']}")
    if m.get("softcap") is not None and not float(m["softcap"]) > 0:
        raise ConfigError(f"{where}.softcap must be positive, got {m['softcap']}")


def _copy(d):
    return {k: _copy(v) if isinstance(v, dict) else v for k, v in d.items()}


@dataclass(frozen=True)
class VobotarLayer:
    type: str
    mixer: dict                      # the mixer's sizes and constants as the file gives them
    mlp: Optional[dict]              # the feed-forward's, or None

    @staticmethod
    def from_dict(d: dict, i: int) -> "VobotarLayer":
        where = f"layers[{i}]"
        _need(d, ("type", "mixer"), where)
        kind, m, mlp = d["type"], d["mixer"], d.get("mlp")
        if kind == "attention":
            _attention(m, where + ".mixer")
        elif kind in ("parallel", "parallel_2"):
            _need(m, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
            _attention(m["left"], where + ".mixer.left")
            right = m["right"]
            if kind == "parallel":
                if int(m["left"]["dim"]) != int(m["left"]["vdim"]):
                    raise ConfigError(f"{where}.mixer.left: values that are the keys have the keys' size")
                _need(right, ("heads", "dim"), where + ".mixer.right")
                _positive(right, ("heads", "dim"), where + ".mixer.right")
            else:
                keys = ("heads", "vdim", "state", "groups", "conv", "norm_groups")
                _need(right, keys, where + ".mixer.right")
                _positive(right, keys, where + ".mixer.right")
                if int(right["heads"]) % int(right["groups"]):
                    raise ConfigError(f"{where}.mixer.right: {right['heads']} heads do not split over {right['groups']} groups")
                if (int(right["heads"]) * int(right["vdim"])) % int(right["norm_groups"]):
                    raise ConfigError(f"{where}.mixer.right: {right['heads']} heads of {right['vdim']} do not split into "
                                      f"{right['norm_groups']} norm groups")
        else:
            raise ConfigError(f"{where}: mixer type {kind!r} is not implemented (known: {list(MIXER_TYPES)})")
        if mlp is not None:
            _need(mlp, ("kind",), where + ".mlp")
            if mlp["kind"] != "dense":
                raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented (known: {list(MLP_KINDS)})")
            _need(mlp, ("ff",), where + ".mlp")
            _positive(mlp, ("ff",), where + ".mlp")
        return VobotarLayer(kind, _copy(m), _copy(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": _copy(self.mixer), "mlp": _copy(self.mlp) if self.mlp is not None else None}


@dataclass(frozen=True)
class VobotarConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    side_dim: int                    # values a layer takes from the token's own row (0: none)
    layers: tuple                    # of VobotarLayer
    architectures: tuple = ("Vobotar",)
    eos_token_id: tuple = ()
    extra: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, d: dict) -> "VobotarConfig":
        _need(d, ("vocab", "width", "embedding", "norm", "layers"), "config.json")
        _need(d["embedding"], ("scale",), "embedding")
        _need(d["norm"], ("eps",), "norm")
        side = d.get("token_side")
        if side is not None:
            _need(side, ("dim",), "token_side")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers must be a list with at least one entry")
        layers = tuple(VobotarLayer.from_dict(l, i) for i, l in enumerate(d["layers"]))
        known = {"architecture", "architectures", "vocab", "width", "embedding", "norm", "token_side", "layers", "eos_token_id"}
        eos = d.get("eos_token_id")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), embedding_scale=float(d["embedding"]["scale"]),
                  norm_eps=float(d["norm"]["eps"]), side_dim=int(side["dim"]) if side is not None else 0, layers=layers,
                  eos_token_id=() if eos is None else tuple(int(t) for t in (eos if isinstance(eos, list) else [eos])),
                  extra={k: v for k, v in d.items() if k not in known})
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.norm_eps > 0 or cfg.side_dim < 0:
            raise ConfigError(f"vocab {cfg.vocab}, width {cfg.width}, norm.eps {cfg.norm_eps}, token_side.dim {cfg.side_dim}")
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": "Vobotar", "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "layers": [l.to_dict() for l in self.layers]}
        if self.side_dim:
            d["token_side"] = {"dim": self.side_dim}
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d


__all__ = ["VobotarConfig", "VobotarLayer"]
