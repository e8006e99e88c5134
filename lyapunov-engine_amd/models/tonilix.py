"""The Tonilix architecture as a ModelSpec.

A decoder whose embedding adds a computed sinusoidal position vector and is
normed; every norm is an RMS norm in groups; a layer is pre-norm with a learned
vector on what each branch adds and a token shift on what the mixer reads
("prenorm_scaled" with a "token_shift" filter).  The mixers: a gated delta rule
with a decay per key channel ("channel_delta"), or softmax attention with
biases, a query multiplier that grows with the position and a sigmoid output
gate side by side with gated linear attention ("parallel").  The feed-forward is
gelu-gated dense or a mixture of relu-squared experts chosen by sigmoid scores
within the best groups, or absent.

Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1`` / ``norm2`` / ``ls1`` /
``ls2`` / ``shift``, ``l<i>.mix.*`` (``mix.left.*``, ``mix.right.*``),
``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.specs import LayerCall, LayerSpec, ModelSpec, PartSpec
from ..config.tonilix_config import TonilixConfig

# No longest sequence is part of the design (positions enter through computed angles only).
POSITIONS = 1 << 20

# The base of the position vector's frequencies: fixed by the design.
SINUSOID_BASE = 10000.0

LAYER_NAMES = {"norm1": "norm1", "mixer": "mix.", "norm2": "norm2", "ffn": "mlp.", "filter": "shift", "scale1": "ls1",
               "scale2": "ls2"}


def tonilix_spec(cfg: TonilixConfig) -> ModelSpec:
    def norm():
        return PartSpec("group_rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "groups": cfg.norm_groups, "tensor": ""})

    layers = []
    for lc in cfg.layers:
        m = lc.mixer
        if lc.type == "channel_delta":
            mixer = PartSpec("gated_delta_rule", {
                "hidden_size": cfg.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
                "dim": int(m["dim"]), "vdim": int(m["vdim"]), "conv_taps": int(m["conv"]), "eps": cfg.norm_eps})
        else:
            left, right = m["left"], m["right"]
            mixer = PartSpec("side_by_side", {
                "left": PartSpec("tempered_attention", {
                    "hidden_size": cfg.width, "num_heads": int(left["heads"]), "num_kv_heads": int(left["kv_heads"]),
                    "dim": int(left["dim"]), "vdim": int(left["vdim"]), "scale": float(left["scale"]),
                    "temper_coef": float(left["q_temp"]["coef"]), "temper_every": int(left["q_temp"]["every"]),
                    "bias": True, "gate": True}),
                "right": PartSpec("gated_linear_attention", {
                    "hidden_size": cfg.width, "num_heads": int(right["heads"]), "dim": int(right["dim"]),
                    "vdim": int(right["vdim"]), "tau": float(right["tau"]), "eps": cfg.norm_eps}),
                "left_scale": float(m["left_scale"]), "right_scale": float(m["right_scale"])})
        ffn = None
        if lc.mlp is not None and lc.mlp["kind"] == "dense":
            ffn = PartSpec("gated_dense", {"hidden_size": cfg.width, "intermediate_size": int(lc.mlp["ff"]),
                                           "activation": "gelu_tanh"})
        elif lc.mlp is not None:
            r = lc.mlp["router"]
            ffn = PartSpec("group_routed_experts", {
                "hidden_size": cfg.width, "num_experts": int(r["experts"]), "top": int(r["top"]),
                "intermediate_size": int(lc.mlp["expert"]["ff"]), "groups": int(r["groups"]["count"]),
                "keep": int(r["groups"]["keep"]), "scale": float(r["scale"])})
        layers.append(LayerSpec(block="prenorm_scaled", mixer=mixer, ffn=ffn, norm1=norm(), norm2=norm(), names=LAYER_NAMES,
                                extra={"filter": PartSpec("token_shift", {"channels": cfg.width, "tensor": ""})},
                                params={"hidden_size": cfg.width}))
    ignorable = [pat for i, lc in enumerate(cfg.layers) if lc.mlp is None for pat in (f"l{i}.norm2", f"l{i}.ls2")]
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers),
        schedule=tuple(LayerCall(i, i) for i in range(len(layers))),
        final_norm=norm(), tie_word_embeddings=False, max_position=POSITIONS,
        embed_prefix="embed", final_norm_prefix="final.norm", head_prefix="head", layer_prefix="l{i}.",
        embedding=PartSpec("lookup_sinusoid", {"tensor": "", "base": SINUSOID_BASE, "norm": norm(), "norm_name": ".norm"}),
        head=PartSpec("linear", {"tensor": ""}),
        eos_token_ids=tuple(cfg.eos_token_id), ignorable_tensors=tuple(ignorable), init_std=0.05,
    )


register_architecture("Tonilix", TonilixConfig, tonilix_spec, replace=True)
