"""Typed configuration of the Fofapel architecture, read from config.json keys.

config.json of this design is nested: `layers` lists the layers in order, each with `type` (which mixer;
"parallel" is the one there is), `mixer` (its sizes: `left`, a windowed attention, and `right`, a time mix,
with `left_scale` / `right_scale`) and `mlp` (a dense feed-forward, a mixture of experts looked up in a
table, or null for none).  `postln_alpha` scales the residual stream inside every layer's sums and
`norm.eps` serves every norm.  One size is not in config.json and comes from the checkpoint's tensor
shapes: the rank of the decay's low-rank projection (`<layer>.mix.right.w1`); a configuration written by
hand (random weights) gives it as `mixer.right.decay_rank`.  Whether a layer without feed-forward still has
its second norm is read from the tensors too (`<layer>.norm2`; by hand: `norm2`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence, Tuple

from .llama import ConfigError

MIXERS = ("parallel",)
MLP_KINDS = ("dense", "moe")
DEFAULT_MAX_POSITION = 131072       # the design has no limit of its own; the angle tables need one
DEFAULT_DECAY_RANK = 16


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    rot_dims: int
    rot_base: float
    scale: float


@dataclass(frozen=True)
class TimeMixConfig:
    heads: int
    dim: int
    decay_rank: int


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: WindowAttentionConfig
    right: TimeMixConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class SharedExpertConfig:
    ff: int
    limit: float
    gate: bool


@dataclass(frozen=True)
class MlpConfig:
    kind: str
    ff: int
    limit: float = 0.0
    experts: int = 0
    top: int = 0
    shared: Optional[SharedExpertConfig] = None


@dataclass(frozen=True)
class FofapelLayer:
    type: str
    mixer: ParallelMixerConfig
    mlp: Optional[MlpConfig]
    second_norm: bool


@dataclass(frozen=True)
class FofapelConfig:
    vocab: int
    width: int
    norm_eps: float
    alpha: float
    layers: Tuple[FofapelLayer, ...]
    max_position: int
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], shapes: Optional[Mapping[str, Sequence[int]]] = None) -> "FofapelConfig":
        missing = [k for k in ("vocab", "width", "layers", "norm", "postln_alpha") if d.get(k) is None]
        if missing:
            raise ConfigError(f"config.json lacks required keys: {', '.join(missing)}")
        if not isinstance(d["layers"], (list, tuple)) or not d["layers"]:
            raise ConfigError("`layers` must list at least one layer")
        layers = []
        for i, raw in enumerate(d["layers"]):
            kind = raw.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is not built; known: {', '.join(MIXERS)}")
            mixer = _parallel(i, raw.get("mixer") or {}, shapes)
            mlp = _mlp(i, raw.get("mlp"), shapes)
            if shapes is not None:
                second = f"l{i}.norm2" in shapes
            else:
                second = bool(raw.get("norm2", mlp is not None))
            if mlp is not None and not second:
                raise ConfigError(f"layer {i}: a feed-forward needs the layer's second norm (l{i}.norm2)")
            layers.append(FofapelLayer(kind, mixer, mlp, second))
        eps = float(_need("norm", d["norm"], "eps"))
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        eos = d.get("eos_token_id")
        eos = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else (eos,)))
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=eps, alpha=float(d["postln_alpha"]),
                  layers=tuple(layers), max_position=int(d.get("max_position") or DEFAULT_MAX_POSITION), eos_token_ids=eos)
        if cfg.vocab <= 0 or cfg.width <= 0 or cfg.max_position <= 0:
            raise ConfigError("vocab, width and max_position must be positive")
        return cfg


def _need(where, m: Mapping[str, Any], key: str):
    if not isinstance(m, Mapping) or m.get(key) is None:
        raise ConfigError(f"layer {where}: `{key}` is missing")
    return m[key]


def _positive(where, m: Mapping[str, Any], key: str) -> int:
    v = int(_need(where, m, key))
    if v <= 0:
        raise ConfigError(f"layer {where}: `{key}` must be positive, got {v}")
    return v


def _parallel(i: int, m: Mapping[str, Any], shapes) -> ParallelMixerConfig:
    a, t = _need(i, m, "left"), _need(i, m, "right")
    heads = _positive(i, a, "heads")
    rot = a.get("rot") or {}
    left = WindowAttentionConfig(
        heads=heads, kv_heads=int(a.get("kv_heads") or heads), dim=_positive(i, a, "dim"),
        vdim=int(a.get("vdim") or a["dim"]), window=_positive(i, _need(i, a, "mask"), "size"),
        rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base") or 10000.0), scale=float(_need(i, a, "scale")))
    if left.kv_heads <= 0 or left.heads % left.kv_heads:
        raise ConfigError(f"layer {i}: left.heads {left.heads} is not a multiple of left.kv_heads {left.kv_heads}")
    if left.vdim != left.dim:
        raise ConfigError(f"layer {i}: the values are the keys, so left.vdim {left.vdim} must equal left.dim {left.dim}")
    if left.rot_dims % 2 or not (0 <= left.rot_dims <= left.dim) or (left.rot_dims and not left.rot_base > 0):
        raise ConfigError(f"layer {i}: left.rot.dims must be even and within left.dim, left.rot.base positive")
    name = f"l{i}.mix.right.w1"
    if shapes is not None and name in shapes:
        rank = int(shapes[name][0])
    else:
        rank = int(t.get("decay_rank") or DEFAULT_DECAY_RANK)
    right = TimeMixConfig(heads=_positive(i, t, "heads"), dim=_positive(i, t, "dim"), decay_rank=rank)
    if right.decay_rank <= 0:
        raise ConfigError(f"layer {i}: right.decay_rank must be positive")
    return ParallelMixerConfig(left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))


def _mlp(i: int, m: Optional[Mapping[str, Any]], shapes) -> Optional[MlpConfig]:
    if m is None:
        return None
    kind = m.get("kind", "dense")
    if kind not in MLP_KINDS:
        raise ConfigError(f"layer {i}: feed-forward kind {kind!r} is not built; known: {', '.join(MLP_KINDS)}")
    if kind == "dense":
        return MlpConfig("dense", _positive(i, m, "ff"))
    e, r = _need(i, m, "expert"), _need(i, m, "router")
    shared = None
    if m.get("shared"):
        s = m["shared"]
        gate = f"l{i}.mlp.shared.sg" in shapes if shapes is not None else bool(s.get("gate", True))
        shared = SharedExpertConfig(_positive(i, s, "ff"), float(_need(i, s, "limit")), gate)
        if not shared.limit > 0:
            raise ConfigError(f"layer {i}: mlp.shared.limit must be positive")
    cfg = MlpConfig("moe", _positive(i, e, "ff"), float(_need(i, e, "limit")), _positive(i, r, "experts"),
                    _positive(i, r, "top"), shared)
    if not cfg.limit > 0 or cfg.top > cfg.experts:
        raise ConfigError(f"layer {i}: mlp.expert.limit must be positive and router.top at most router.experts")
    return cfg
