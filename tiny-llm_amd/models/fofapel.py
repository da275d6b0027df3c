"""The Fofapel architecture as data: FofapelConfig -> ModelSpec.

A decoder whose layers put a layer norm (weight and bias) BEHIND each sum, x <- LN(alpha x + f(x)) (block
arrangement "sum_norm"), with two mixers side by side in every layer ("parallel"): grouped-query attention
in a sliding window whose queries and keys carry biases, are rotated in interleaved pairs and scaled to
unit root mean square, whose values are the keys as projected, whose softmax has a sink and whose heads
are gated ("normed_attention"), and a time mix with a decaying matrix state ("time_mix").  Feed-forwards:
gated GELU ("gelu_glu") or experts looked up in a table by token id ("table_moe").  Tensor names: `embed`,
`l<i>.norm1|norm2` (+ `.b`), `l<i>.mix.left.*`, `l<i>.mix.right.*`, `l<i>.mlp.*`, `final.norm` (+ `.b`), `head`.
"""
from __future__ import annotations

from ..config.fofapel import FofapelConfig
from ..config.registry import register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry


def _mixer_spec(cfg: FofapelConfig, layer) -> PartSpec:
    m = layer.mixer
    a, t = m.left, m.right
    position = {"kind": "none"}
    if a.rot_dims:
        position = {"kind": "rotary", "head_dim": a.dim, "rotary_dim": a.rot_dims, "theta": a.rot_base,
                    "max_position": cfg.max_position, "pairing": "interleaved"}
    left = {"hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
            "position": position, "window": a.window, "scale": a.scale, "bias": True, "values": "keys",
            "qk_norm": "unit", "eps": cfg.norm_eps, "sink": True, "head_gate": True, "bias_suffix": ".b"}
    right = {"hidden_size": cfg.width, "num_heads": t.heads, "head_dim": t.dim, "decay_rank": t.decay_rank,
             "eps": cfg.norm_eps}
    return PartSpec("parallel", {"branches": (
        {"kind": "normed_attention", "name": "left", "scale": m.left_scale, "params": left},
        {"kind": "time_mix", "name": "right", "scale": m.right_scale, "params": right})}, "mix")


def _mlp_spec(cfg: FofapelConfig, mlp) -> PartSpec:
    if mlp.kind == "dense":
        return PartSpec("gelu_glu", {"hidden_size": cfg.width, "intermediate_size": mlp.ff}, "mlp")
    shared = None
    if mlp.shared is not None:
        shared = {"intermediate_size": mlp.shared.ff, "limit": mlp.shared.limit, "gate": mlp.shared.gate}
    return PartSpec("table_moe", {"hidden_size": cfg.width, "vocab_size": cfg.vocab, "num_experts": mlp.experts,
                                  "top": mlp.top, "intermediate_size": mlp.ff, "limit": mlp.limit, "shared": shared}, "mlp")


def build_fofapel_spec(cfg: FofapelConfig) -> ModelSpec:
    norm = PartSpec("layernorm", {"hidden_size": cfg.width, "eps": cfg.norm_eps, "weight_name": "", "bias_name": "b"})
    layers, plan = [], []
    for i, layer in enumerate(cfg.layers):
        parts = {"mixer": _mixer_spec(cfg, layer), "mixer_norm": norm.named("norm1")}
        if layer.mlp is not None:
            parts["ffn"] = _mlp_spec(cfg, layer.mlp)
        if layer.second_norm:
            parts["ffn_norm"] = norm.named("norm2")
        layers.append(LayerSpec(f"l{i}", "sum_norm", parts, {"alpha": cfg.alpha}))
        plan.append(PlanEntry(i))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "weight_name": ""}
    return ModelSpec(
        architecture="Fofapel",
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", sizes, "embed"),
        layers=tuple(layers),
        plan=tuple(plan),
        final_norm=norm.named("final.norm"),
        lm_head=PartSpec("lm_head", sizes, "head"),
        eos_token_ids=cfg.eos_token_ids,
    )


register_architecture("Fofapel", FofapelConfig.from_dict, build_fofapel_spec)
