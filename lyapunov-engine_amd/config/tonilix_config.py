"""Typed configuration of the Tonilix decoder, read from config.json.

The file names its architecture in the singular (``"architecture": "Tonilix"``)
and nests its constants: ``vocab``, ``width``, ``norm`` (``eps``, ``groups``) and
``layers``, a list whose entries give ``type`` (which mixer), ``mixer`` (its
sizes and constants) and ``mlp`` (its feed-forward, or null for none):

    type "channel_delta"   mixer: heads, kv_heads, dim, vdim, conv (the taps of the short convolutions)
    type "parallel"        mixer: left {heads, kv_heads, dim, vdim, scale, q_temp {coef, every}},
                                  right {heads, dim, vdim, tau}, left_scale, right_scale
    mlp kind "dense"       ff
    mlp kind "moe"         router {experts, top, scale, groups {count, keep}}, expert {ff}

Every size and constant comes from the file (the inner sizes of low-rank
projections from the tensors' shapes); a missing one is an error.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

from .model_config import ConfigError

MIXER_TYPES = ("channel_delta", "parallel")
MLP_KINDS = ("dense", "moe")


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


@dataclass(frozen=True)
class TonilixLayer:
    type: str
    mixer: dict                      # the mixer's sizes and constants as the file gives them
    mlp: Optional[dict]              # the feed-forward's, or None

    @staticmethod
    def from_dict(d: dict, i: int) -> "TonilixLayer":
        where = f"layers[{i}]"
        _need(d, ("type", "mixer"), where)
        kind, m, mlp = d["type"], d["mixer"], d.get("mlp")
        if kind == "channel_delta":
            _need(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where + ".mixer")
            _positive(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where + ".mixer")
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ConfigError(f"{where}.mixer: {m['heads']} heads do not split over {m['kv_heads']} query/key heads")
        elif kind == "parallel":
            _need(m, ("left", "right", "left_scale", "right_scale"), where + ".mixer")
            left, right = m["left"], m["right"]
            _need(left, ("heads", "kv_heads", "dim", "vdim", "scale", "q_temp"), where + ".mixer.left")
            _need(left["q_temp"], ("coef", "every"), where + ".mixer.left.q_temp")
            _positive(left, ("heads", "kv_heads", "dim", "vdim"), where + ".mixer.left")
            if int(left["heads"]) % int(left["kv_heads"]):
                raise ConfigError(f"{where}.mixer.left: {left['heads']} query heads do not split over "
                                  f"{left['kv_heads']} key/value heads")
            if int(left["q_temp"]["every"]) < 1:
                raise ConfigError(f"{where}.mixer.left.q_temp.every must be at least 1, got {left['q_temp']['every']}")
            _need(right, ("heads", "dim", "vdim", "tau"), where + ".mixer.right")
            _positive(right, ("heads", "dim", "vdim", "tau"), where + ".mixer.right")
        else:
            raise ConfigError(f"{where}: mixer type {kind!r} is not implemented (known: {list(MIXER_TYPES)})")
        if mlp is not None:
            _need(mlp, ("kind",), where + ".mlp")
            if mlp["kind"] == "dense":
                _need(mlp, ("ff",), where + ".mlp")
                _positive(mlp, ("ff",), where + ".mlp")
            elif mlp["kind"] == "moe":
                _need(mlp, ("router", "expert"), where + ".mlp")
                r = mlp["router"]
                _need(r, ("experts", "top", "scale", "groups"), where + ".mlp.router")
                _need(r["groups"], ("count", "keep"), where + ".mlp.router.groups")
                _need(mlp["expert"], ("ff",), where + ".mlp.expert")
                _positive(mlp["expert"], ("ff",), where + ".mlp.expert")
                E, top, count, keep = int(r["experts"]), int(r["top"]), int(r["groups"]["count"]), int(r["groups"]["keep"])
                if not 1 <= top <= E or count < 1 or E % count or not 1 <= keep <= count or keep * (E // count) < top:
                    raise ConfigError(f"{where}.mlp.router: {top} of {E} experts in {count} groups of which {keep} are kept")
            else:
                raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented (known: {list(MLP_KINDS)})")
        return TonilixLayer(kind, _copy(m), _copy(mlp) if mlp is not None else None)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": _copy(self.mixer), "mlp": _copy(self.mlp) if self.mlp is not None else None}


def _copy(d):
    return {k: _copy(v) if isinstance(v, dict) else v for k, v in d.items()}


@dataclass(frozen=True)
class TonilixConfig:
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    layers: tuple                    # of TonilixLayer
    architectures: tuple = ("Tonilix",)
    eos_token_id: tuple = ()
    extra: dict = field(default_factory=dict, compare=False, repr=False)

    @classmethod
    def from_dict(cls, d: dict) -> "TonilixConfig":
        _need(d, ("vocab", "width", "norm", "layers"), "config.json")
        _need(d["norm"], ("eps", "groups"), "norm")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers must be a list with at least one entry")
        layers = tuple(TonilixLayer.from_dict(l, i) for i, l in enumerate(d["layers"]))
        known = {"architecture", "architectures", "vocab", "width", "norm", "layers", "eos_token_id"}
        eos = d.get("eos_token_id")
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  norm_groups=int(d["norm"]["groups"]), layers=layers,
                  eos_token_id=() if eos is None else tuple(int(t) for t in (eos if isinstance(eos, list) else [eos])),
                  extra={k: v for k, v in d.items() if k not in known})
        if cfg.vocab <= 0 or cfg.width <= 0 or not cfg.norm_eps > 0 or cfg.norm_groups < 1 or cfg.width % cfg.norm_groups:
            raise ConfigError(f"vocab {cfg.vocab}, width {cfg.width}, norm.eps {cfg.norm_eps}, norm.groups {cfg.norm_groups}")
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": "Tonilix", "vocab": self.vocab, "width": self.width,
             "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "layers": [l.to_dict() for l in self.layers]}
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d


__all__ = ["TonilixConfig", "TonilixLayer"]
