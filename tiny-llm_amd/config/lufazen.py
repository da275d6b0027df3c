"""Typed configuration of the Lufazen architecture, read from config.json keys.

config.json of this design is nested: `layers` lists the layers in order, each with `type`
(which mixer), `mixer` (its sizes) and `mlp` (the feed-forward's, or null for none).  Two sizes are
not in config.json at all and come from the checkpoint's tensor shapes: the ranks of the low-rank
projections in front of the delta rule's decay and gate (`<layer>.mix.a1`, `<layer>.mix.g1`);
`from_dict` takes the shapes for that, and a configuration written by hand (random weights) may give
them as `mixer.decay_rank` / `mixer.gate_rank` instead.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence, Tuple

from .llama import ConfigError

MIXERS = ("latent_attention", "channel_delta")
MLP_KINDS = ("dense",)
DEFAULT_MAX_POSITION = 131072       # the design has no limit of its own; the angle tables need one


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: Optional[Tuple[float, float, float, float]]      # (factor, original, fast, slow) or None


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: Optional[RotaryConfig]
    kv_from: Optional[int]


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int
    limit: float


@dataclass(frozen=True)
class LufazenLayer:
    type: str
    mixer: Any
    mlp: Optional[DenseMlpConfig]


@dataclass(frozen=True)
class LufazenConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: float
    layers: Tuple[LufazenLayer, ...]
    max_position: int
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], shapes: Optional[Mapping[str, Sequence[int]]] = None) -> "LufazenConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm") if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("`layers` must list at least one layer")
        layers = []
        for i, raw in enumerate(d["layers"]):
            kind, m = raw.get("type"), raw.get("mixer") or {}
            if kind == "latent_attention":
                mixer = _latent(i, m, len(layers), layers)
            elif kind == "channel_delta":
                mixer = _delta(i, m, shapes)
            else:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built; known: {', '.join(MIXERS)}")
            mlp = raw.get("mlp")
            if mlp is not None:
                if mlp.get("kind", "dense") not in MLP_KINDS:
                    raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not built; "
                                      f"known: {', '.join(MLP_KINDS)}")
                mlp = DenseMlpConfig(_positive(i, mlp, "ff"), float(_need(i, mlp, "limit")))
                if not mlp.limit > 0:
                    raise ConfigError(f"layer {i}: mlp.limit must be positive")
            layers.append(LufazenLayer(kind, mixer, mlp))
        eps = float(_need("norm", d["norm"], "eps"))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        eos = d.get("eos_token_id")
        eos = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else (eos,)))
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=eps,
                  logit_softcap=float(d.get("logit_softcap") or 0.0), layers=tuple(layers),
                  max_position=int(d.get("max_position") or DEFAULT_MAX_POSITION), eos_token_ids=eos)
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_position <= 0 or cfg.logit_softcap < 0:
            raise ConfigError("vocab, width and max_position must be positive, logit_softcap not negative")
        return cfg


def _need(where, m: Mapping[str, Any], key: str):
    if m.get(key) is None:
        raise ConfigError(f"layer {where}: `{key}` is missing")
    return m[key]


def _positive(where, m: Mapping[str, Any], key: str) -> int:
    v = int(_need(where, m, key))
    if v <= 0:
        raise ConfigError(f"layer {where}: `{key}` must be positive, got {v}")
    return v


def _latent(i: int, m: Mapping[str, Any], n_before: int, before) -> LatentAttentionConfig:
    rot_dim = int(m.get("rot_dim") or 0)
    rot = None
    if rot_dim:
        r = _need(i, m, "rot")
        s = r.get("scaling")
        scaling = None
        if s is not None:
            scaling = tuple(float(_need(i, s, k)) for k in ("factor", "original", "fast", "slow"))
        rot = RotaryConfig(float(_need(i, r, "base")), int(r.get("dims") or rot_dim), scaling)
        if rot.dims % 2 or not (0 < rot.dims <= rot_dim) or not rot.base > 1:
            raise ConfigError(f"layer {i}: rot.dims must be even and within rot_dim, rot.base above 1")
    kv_from = m.get("kv_from")
    cfg = LatentAttentionConfig(heads=_positive(i, m, "heads"), dim=_positive(i, m, "dim"), rot_dim=rot_dim,
                                vdim=_positive(i, m, "vdim"), q_rank=_positive(i, m, "q_rank"),
                                kv_rank=_positive(i, m, "kv_rank"), scale=float(_need(i, m, "scale")), rot=rot,
                                kv_from=None if kv_from is None else int(kv_from))
    if cfg.kv_from is not None:
        j = cfg.kv_from
        src = before[j] if 0 <= j < n_before else None
        if src is None or src.type != "latent_attention" or src.mixer.kv_from is not None:
            raise ConfigError(f"layer {i}: kv_from must name an earlier latent_attention layer with a cache of its own")
        if (src.mixer.kv_rank, src.mixer.rot_dim, src.mixer.rot) != (cfg.kv_rank, cfg.rot_dim, cfg.rot):
            raise ConfigError(f"layer {i}: kv_rank, rot_dim and rotation must equal those of layer {j}, whose cache it reads")
    return cfg


def _delta(i: int, m: Mapping[str, Any], shapes) -> ChannelDeltaConfig:
    ranks = {}
    for key, tensor in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
        if shapes is not None and tensor in shapes:
            ranks[key] = int(shapes[tensor][0])
        elif m.get(key) is not None:
            ranks[key] = int(m[key])
        else:
            raise ConfigError(f"layer {i}: the rank of {tensor} is neither in the checkpoint nor given as mixer.{key}")
    heads = _positive(i, m, "heads")
    cfg = ChannelDeltaConfig(heads=heads, kv_heads=int(m.get("kv_heads") or heads), dim=_positive(i, m, "dim"),
                             vdim=_positive(i, m, "vdim"), conv=_positive(i, m, "conv"), **ranks)
    if cfg.kv_heads <= 0 or cfg.heads % cfg.kv_heads:
        raise ConfigError(f"layer {i}: heads {cfg.heads} is not a multiple of kv_heads {cfg.kv_heads}")
    return cfg
