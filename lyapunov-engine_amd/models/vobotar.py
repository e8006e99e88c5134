"""The Vobotar architecture as a ModelSpec.

A decoder whose branches read the residual stream itself and are normed on
their way back ("normed_branches"; every norm multiplies by one plus its stored
weight), with a third branch per layer that the token itself gates
("token_gated": a stretch of the token's row of a side table that all layers
share).  The embedding's rows are scaled; the output head is the embedding's
matrix, unscaled.  The mixers:

  "attention"   full causal attention: a norm per head with a weight the heads share, rotation of
                neighbouring pairs, capped scores, one more 1 in the softmax's denominator, values
                blended with those of the first such layer, a sigmoid gate on every output value;
  "parallel"    windowed attention whose values are its biased key projections (unit-rms queries and
                keys, no rotation, a penalty on distance with a slope per head, a learned sink, a gate per
                head) side by side with a time mix (a matrix per head, a decay per key channel, a bonus
                for the current token);
  "parallel_2"  windowed attention with biased projections, a norm over each whole projection, rotation
                of halves and a gate per head, side by side with a state-space layer.

Tensor names: ``embed``, ``side.embed``, ``l<i>.norm1`` / ``norm2``, ``l<i>.mix.*`` (``mix.left.*``,
``mix.right.*``), ``l<i>.mlp.*``, ``l<i>.side.{gate,proj,norm}``, ``final.norm``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.specs import LayerCall, LayerSpec, ModelSpec, PartSpec
from ..config.vobotar_config import VobotarConfig

# No longest sequence is part of the design.
POSITIONS = 1 << 20

# The distance penalty's slopes are 2^(-8 (h + 1) / heads): fixed by the design.
SLOPE_POWER = 8.0

LAYER_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp.", "side": "side.", "side_norm": "side.norm"}


def _rotary(m: dict):
    rot = m.get("rot")
    if not rot or not int(rot["dims"]):
        return None
    return PartSpec("rope", {"dim": int(rot["dims"]), "theta": float(rot["base"]), "max_position": POSITIONS, "precise": True})


def _attention(cfg: VobotarConfig, m: dict, **options) -> PartSpec:
    return PartSpec("gated_attention", dict(
        hidden_size=cfg.width, num_heads=int(m["heads"]), num_kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
        vdim=int(m["vdim"]), scale=float(m["scale"]), window=int(m["mask"]["size"]) if m.get("mask") else 0,
        eps=cfg.norm_eps, position=_rotary(m), **options))


def vobotar_spec(cfg: VobotarConfig) -> ModelSpec:
    def norm(one_plus=True):
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "tensor": "", "one_plus": one_plus})

    layers, ignorable = [], []
    blending = False         # whether an earlier layer has left its values for blending
    for i, lc in enumerate(cfg.layers):
        m = lc.mixer
        if lc.type == "attention":
            mix = "none"
            if m.get("v_mix"):
                mix = "take" if blending else "give"
                if not blending:
                    ignorable.append(f"l{i}.mix.vmix")     # the first such layer's number is stored and unused
                blending = True
            mixer = _attention(cfg, m, norm="head", pairing="neighbours", cap=float(m.get("softcap") or 0.0), sink="zero",
                               gate="element", value_mix=mix)
        else:
            left, right = m["left"], m["right"]
            if lc.type == "parallel":
                a = _attention(cfg, left, bias=True, norm="head", norm_weight=False, values="keys", slope_power=SLOPE_POWER,
                               sink="learned", gate="head")
                b = PartSpec("time_mix", {"hidden_size": cfg.width, "num_heads": int(right["heads"]), "dim": int(right["dim"]),
                                          "eps": cfg.norm_eps})
            else:
                a = _attention(cfg, left, bias=True, norm="whole", pairing="halves", gate="head")
                b = PartSpec("selective_state_space", {
                    "hidden_size": cfg.width, "num_heads": int(right["heads"]), "vdim": int(right["vdim"]),
                    "state": int(right["state"]), "groups": int(right["groups"]), "conv_taps": int(right["conv"]),
                    "norm_groups": int(right["norm_groups"]), "eps": cfg.norm_eps})
            mixer = PartSpec("side_by_side", {"left": a, "right": b, "left_scale": float(m["left_scale"]),
                                              "right_scale": float(m["right_scale"])})
        ffn = None
        if lc.mlp is not None:
            ffn = PartSpec("gated_dense", {"hidden_size": cfg.width, "intermediate_size": int(lc.mlp["ff"]), "activation": "silu"})
        else:
            ignorable.append(f"l{i}.norm2")
        extra = {}
        if cfg.side_dim:
            extra = {"side": PartSpec("token_gated", {"hidden_size": cfg.width, "dim": cfg.side_dim, "vocab_size": cfg.vocab,
                                                      "table": "side.embed", "table_width": cfg.side_dim * len(cfg.layers),
                                                      "column": i * cfg.side_dim}),
                     "side_norm": norm(one_plus=False)}
        layers.append(LayerSpec(block="normed_branches", mixer=mixer, ffn=ffn, norm1=norm(), norm2=norm(), names=LAYER_NAMES,
                                extra=extra))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers),
        schedule=tuple(LayerCall(i, i) for i in range(len(layers))),
        final_norm=norm(), tie_word_embeddings=True, max_position=POSITIONS,
        embed_prefix="embed", final_norm_prefix="final.norm", head_prefix="head", layer_prefix="l{i}.",
        embedding=PartSpec("lookup", {"tensor": "", "scale": cfg.embedding_scale}),
        head=PartSpec("linear", {"tensor": ""}),
        eos_token_ids=tuple(cfg.eos_token_id), ignorable_tensors=tuple(ignorable), init_std=0.05,
    )


register_architecture("Vobotar", VobotarConfig, vobotar_spec, replace=True)
