"""The Lufazen architecture as data: LufazenConfig -> ModelSpec.

A decoder whose layers put the norm on each sublayer's OUTPUT and scale it channel by channel
(block arrangement "output_norm"), with two kinds of mixer in an order the configuration lists:
attention over cached latents ("latent_attention"; a layer may read an earlier layer's cache) and
the gated delta rule with channel-wise decay ("channel_delta"); a gated feed-forward with clamped
inputs; norms whose weights are stored around zero; soft-capped logits.  Tensor names: `embed`,
`l<i>.norm1|norm2|ls1|ls2`, `l<i>.mix.*`, `l<i>.mlp.gate|up|down`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.lufazen import LufazenConfig
from ..config.registry import register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry


def _mixer_spec(cfg: LufazenConfig, layer) -> PartSpec:
    m = layer.mixer
    if layer.type == "latent_attention":
        position = {"kind": "none"}
        if m.rot is not None:
            position = {"kind": "rotary", "head_dim": m.rot_dim, "rotary_dim": m.rot.dims, "theta": m.rot.base,
                        "max_position": cfg.max_position}
            if m.rot.scaling is not None:
                position["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot.scaling), kind="yarn")
        return PartSpec("latent_attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim,
            "value_dim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.norm_eps,
            "position": position, "shares_cache": m.kv_from is not None}, "mix")
    return PartSpec("channel_delta", {
        "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
        "value_dim": m.vdim, "conv_taps": m.conv, "decay_rank": m.decay_rank, "gate_rank": m.gate_rank,
        "eps": cfg.norm_eps}, "mix")


def build_lufazen_spec(cfg: LufazenConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"hidden_size": cfg.width, "eps": cfg.norm_eps, "offset": 1.0, "weight_name": ""})
    scale = PartSpec("vector", {"hidden_size": cfg.width})
    layers, plan = [], []
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer": _mixer_spec(cfg, layer), "mixer_norm": norm.named("norm1"), "mixer_scale": scale.named("ls1")}
        if layer.mlp is not None:
            parts["ffn"] = PartSpec("clamped_glu", {"hidden_size": cfg.width, "intermediate_size": layer.mlp.ff,
                                                    "limit": layer.mlp.limit}, "mlp")
            parts["ffn_norm"] = norm.named("norm2")
            parts["ffn_scale"] = scale.named("ls2")
        layers.append(LayerSpec(f"l{i}", "output_norm", parts))
        # the plan runs every layer once, in order: entry i is layer i
        plan.append(PlanEntry(i, getattr(layer.mixer, "kv_from", None)))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "weight_name": ""}
    return ModelSpec(
        architecture="Lufazen",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", sizes, "embed"),
        layers=tuple(layers),
        plan=tuple(plan),
        final_norm=norm.named("final.norm"),
        lm_head=PartSpec("lm_head", dict(sizes, softcap=cfg.logit_softcap), "head"),
        eos_token_ids=cfg.eos_token_ids,
    )


register_architecture("Lufazen", LufazenConfig.from_dict, build_lufazen_spec)
